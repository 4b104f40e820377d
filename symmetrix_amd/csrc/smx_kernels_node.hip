// Node-level kernels for gfx950: symmetric contraction, MFMA channel mixing,
// readout tail, integer list preparation and caller-side force reduction.
#include "smx_device.hpp"
#include "smx_kernels.hpp"
#include "smx_host_model.hpp"

#include <algorithm>

namespace smx {

// ===========================================================================
// Integer list preparation
namespace {

constexpr int SCAN_BLOCK = 1024;

// exclusive scan of one 1024-element tile held by a 1024-thread block
__device__ int block_scan_exclusive(int v, int* total)
{
    __shared__ int wsum[16];
    const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int t = __shfl_up(incl, off, 64);
        if (lane >= off) incl += t;
    }
    if (lane == 63) wsum[w] = incl;
    __syncthreads();
    if (w == 0) {
        int s = lane < 16 ? wsum[lane] : 0;
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) {
            const int t = __shfl_up(s, off, 64);
            if (lane >= off) s += t;
        }
        if (lane < 16) wsum[lane] = s;
    }
    __syncthreads();
    const int base = w ? wsum[w - 1] : 0;
    *total = wsum[15];
    __syncthreads();
    return base + incl - v;
}

__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_tiles(const int* in, int* out, int n, int* block_sums)
{
    const int i = blockIdx.x * SCAN_BLOCK + threadIdx.x;
    const int v = i < n ? in[i] : 0;
    int total;
    const int ex = block_scan_exclusive(v, &total);
    if (i < n) out[i] = ex;
    if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}
// scan of the per-tile sums (up to 1024 tiles per pass, looped) and write of out[n]
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_sums(int* block_sums, int nb, int* out, int n)
{
    int carry = 0;
    for (int b0 = 0; b0 < nb; b0 += SCAN_BLOCK) {
        const int i = b0 + threadIdx.x;
        const int v = i < nb ? block_sums[i] : 0;
        int total;
        const int ex = block_scan_exclusive(v, &total);
        if (i < nb) block_sums[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) out[n] = carry;
}
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_add(int* out, int n, const int* block_sums)
{
    const int i = blockIdx.x * SCAN_BLOCK + threadIdx.x;
    if (i < n) out[i] += block_sums[blockIdx.x];
}

// keys outside [0, rows) are ignored (callers that hand over device arrays are not range-checked)
__global__ void k_count(const int* key, long n, int rows, int* count)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int j = key[i];
        if (j >= 0 && j < rows) atomicAdd(&count[j], 1);
    }
}
__global__ void k_place(const int* key, long n, int rows, const int* start, int* cursor, int* list)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int j = key[i];
        if (j >= 0 && j < rows) list[start[j] + atomicAdd(&cursor[j], 1)] = (int)i;
    }
}
// Ascending order inside every bucket (the atomic placement above is unordered).
// One wavefront per bucket; entries are distinct, so the rank of an entry is the
// number of smaller ones: bucket staged in LDS, every lane counts for its entries.
constexpr int SORT_LDS = 1024;
// The bucket's counter and cursor are dead by now: they are cleared here, so that the next list build
// finds them at zero without a launch of its own.
// With a guard (device-resident callers, whose arrays no host code has looked at): when the checks of this
// evaluation raised its status word, the CSR offsets and the species groups are set to "no edges, no nodes", so
// that no later kernel of the evaluation uses an unchecked integer as an address; the status goes into the sticky
// word the host reads at its next synchronising call and, raised or not, into the word the later kernels read.
__global__ __launch_bounds__(64) void k_sort_buckets(const int* start, int rows, int* list, int* count, int* cursor,
                                                     InputGuard g)
{
    __shared__ int buf[SORT_LDS];
    const int j = blockIdx.x;
    if (g.status) {
        const int st = *g.status;
        if (st) {
            for (int i = j * 64 + threadIdx.x; i < g.n_first; i += gridDim.x * 64) g.first_neigh[i] = 0;
            for (int i = j * 64 + threadIdx.x; i < g.n_tstart; i += gridDim.x * 64) g.tstart[i] = 0;
            if (j == 0 && threadIdx.x == 0) atomicOr(g.sticky, st);
        }
        if (j == 0 && threadIdx.x == 0) *g.live = st;
    }
    if (threadIdx.x == 0) { count[j] = 0; cursor[j] = 0; }
    const int s0 = start[j], n = start[j + 1] - s0;
    if (n <= 1) return;
    if (n <= SORT_LDS) {
        for (int t = threadIdx.x; t < n; t += 64) buf[t] = list[s0 + t];
        __syncthreads();
        for (int t = threadIdx.x; t < n; t += 64) {
            const int v = buf[t];
            int rank = 0;
            for (int q = 0; q < n; ++q) rank += buf[q] < v;
            list[s0 + rank] = v;
        }
    } else if (threadIdx.x == 0) {
        // very long bucket: in-place insertion sort by one lane (correct, slow, not expected in practice)
        for (int a = s0 + 1; a < s0 + n; ++a) {
            const int v = list[a];
            int b = a - 1;
            while (b >= s0 && list[b] > v) { list[b + 1] = list[b]; --b; }
            list[b + 1] = v;
        }
    }
}
// species groups in one block: LDS histogram, scan over the (few) species, placement
__device__ void type_groups_body(const int* node_types, int N, int T, int* tstart, int* perm, int* sh)
{
    // sh: [T] counts, [T] cursors
    int* cnt = sh;
    int* cur = sh + T;
    for (int t = threadIdx.x; t < T; t += blockDim.x) { cnt[t] = 0; cur[t] = 0; }
    __syncthreads();
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        const int t = node_types[i];
        if (t >= 0 && t < T) atomicAdd(&cnt[t], 1);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        int acc = 0;
        for (int t = 0; t < T; ++t) { const int c = cnt[t]; cnt[t] = acc; tstart[t] = acc; acc += c; }
        tstart[T] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < N; i += blockDim.x) {
        const int t = node_types[i];
        if (t >= 0 && t < T) perm[cnt[t] + atomicAdd(&cur[t], 1)] = i;
    }
}
__global__ __launch_bounds__(1024) void k_type_groups(const int* node_types, int N, int T, int* tstart, int* perm)
{
    extern __shared__ int sh[];
    type_groups_body(node_types, N, T, tstart, perm, sh);
}
// Receivers in order of decreasing degree (counting sort on min(degree, 1023), one block).  The edge
// kernels hand consecutive entries to the rows of a wavefront, which then finish together; the order
// inside a degree class is whatever the LDS atomics leave and has no influence on any result.
// `v` holds the CSR offsets (counts == false) or the degrees themselves (counts == true).
__device__ void degree_order_body(int N, const int* v, int* order, bool counts = false)
{
    __shared__ int start[1024];
    __shared__ int cur[1024];
    __shared__ int wsum[16];
    const int tid = threadIdx.x;
    start[tid] = 0; cur[tid] = 0;
    __syncthreads();
    for (int i = tid; i < N; i += 1024) {
        const int d = min(max(counts ? v[i] : v[i + 1] - v[i], 0), 1023);   // a negative count must not index below the table
        atomicAdd(&start[1023 - d], 1);
    }
    __syncthreads();
    // exclusive scan of the 1024 counts: wavefront scans, then the 16 wavefront totals
    const int c = start[tid];
    int incl = c;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int o = __shfl_up(incl, off, 64);
        if ((tid & 63) >= off) incl += o;
    }
    if ((tid & 63) == 63) wsum[tid >> 6] = incl;
    __syncthreads();
    int base = 0;
    for (int w = 0; w < (tid >> 6); ++w) base += wsum[w];
    __syncthreads();
    start[tid] = base + incl - c;
    __syncthreads();
    for (int i = tid; i < N; i += 1024) {
        const int b = 1023 - min(max(counts ? v[i] : v[i + 1] - v[i], 0), 1023);
        order[start[b] + atomicAdd(&cur[b], 1)] = i;
    }
}
__global__ __launch_bounds__(1024) void k_degree_order(int N, const int* first_neigh, int* order)
{
    degree_order_body(N, first_neigh, order);
}
__global__ void k_check_range(const int* v, long n, int limit, int* flags)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && (v[i] < 0 || v[i] >= limit)) atomicOr(flags, 1);
}
__global__ void k_check_r(const double* r, long n, double r_cut, int* flags)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && !(r[i] > 0.0 && r[i] < r_cut)) atomicOr(flags, 2);
}
template <typename T>
__global__ void k_fill(T* p, long n, T v)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = v;
}
template <typename TS, typename TD>
__global__ void k_convert(const TS* s, TD* d, long n)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) d[i] = (TD)s[i];
}
inline unsigned nblk(long n, int bs) { return (unsigned)((n + bs - 1) / bs); }

// whole scan in one block (tiles visited in order with a running carry): one launch
// instead of three while the array is short
__device__ void scan_single_body(const int* in, int* out, int n)
{
    int carry = 0;
    for (int b0 = 0; b0 < n; b0 += SCAN_BLOCK) {
        const int i = b0 + threadIdx.x;
        const int v = i < n ? in[i] : 0;
        int total;
        const int ex = block_scan_exclusive(v, &total);
        if (i < n) out[i] = carry + ex;
        carry += total;
    }
    if (threadIdx.x == 0) out[n] = carry;
}
__global__ __launch_bounds__(SCAN_BLOCK) void k_scan_single(const int* in, int* out, int n)
{
    scan_single_body(in, out, n);
}
// The node-level lists of one evaluation in one launch (one block): first_neigh = exclusive scan of
// num_neigh, receivers by decreasing degree, species groups, and the zeroing of `zero_n` counters that the
// sender-list kernels count into.  Each part is the body of the stand-alone kernel of the same name.
__global__ __launch_bounds__(SCAN_BLOCK) void k_node_lists(const int* num_neigh, int N, int* first_neigh, int* order,
                                                          const int* node_types, int T, int* tstart, int* perm,
                                                          int* zero_p, long zero_n)
{
    extern __shared__ int sh[];
    for (long i = threadIdx.x; i < zero_n; i += SCAN_BLOCK) zero_p[i] = 0;
    scan_single_body(num_neigh, first_neigh, N);
    __syncthreads();   // first_neigh, written by this block, is read back below
    degree_order_body(N, first_neigh, order);
    __syncthreads();
    type_groups_body(node_types, N, T, tstart, perm, sh);
}
// The same with the sender histogram in the same launch: blocks 0, 1, 2 form one node list each, the other blocks
// count the senders (counters at zero on entry), which does not depend on the node lists.
// With `chk.status` set the launch also checks everything the later kernels use as an address or a table argument
// (species, sender rows, edge lengths, counts that add up to the edge totals) and raises bits in the status word.
__global__ __launch_bounds__(SCAN_BLOCK) void k_node_lists_count(const int* num_neigh, int N, int* first_neigh, int* order,
                                                                const int* node_types, int T, int* tstart, int* perm,
                                                                const int* key, long n, int rows, int* count, int* rank,
                                                                InputChecks chk)
{
    extern __shared__ int sh[];
    // the three node lists are independent of each other: a block each
    if (blockIdx.x == 0) {
        scan_single_body(num_neigh, first_neigh, N);
        __syncthreads();   // first_neigh, written by this block, is read back below
        if (chk.status) {
            int bad = 0;
            for (int i = threadIdx.x; i < N; i += SCAN_BLOCK) bad |= (num_neigh[i] < 0) | (node_types[i] < 0) | (node_types[i] >= T);
            if (threadIdx.x == 0) bad |= (first_neigh[N] != (int)chk.num_edges) | (first_neigh[chk.num_local_nodes] != (int)n);
            if (bad) atomicOr(chk.status, 1);
        }
        return;
    }
    if (blockIdx.x == 1) { degree_order_body(N, num_neigh, order, true); return; }
    if (blockIdx.x == 2) { type_groups_body(node_types, N, T, tstart, perm, sh); return; }
    constexpr int LIST_BLOCKS = 3;
    for (long i = (long)(blockIdx.x - LIST_BLOCKS) * SCAN_BLOCK + threadIdx.x; i < n; i += (long)(gridDim.x - LIST_BLOCKS) * SCAN_BLOCK) {
        const int j = key[i];
        if (j >= 0 && j < rows) rank[i] = atomicAdd(&count[j], 1);   // the entry's place inside its bucket
        else if (chk.status) atomicOr(chk.status, 1);
    }
    if (chk.status) {
        // species and length of every edge (layer 0 covers the edges of ghost receivers as well)
        int bad = 0;
        for (long i = (long)(blockIdx.x - LIST_BLOCKS) * SCAN_BLOCK + threadIdx.x; i < chk.num_edges; i += (long)(gridDim.x - LIST_BLOCKS) * SCAN_BLOCK) {
            const int t = chk.neigh_types[i];
            const double rr = chk.r[i];
            bad |= (t < 0 || t >= T) ? 1 : 0;
            bad |= (rr > 0.0 && rr < chk.r_cut) ? 0 : 2;
        }
        if (bad) atomicOr(chk.status, bad);
    }
}
// the same checks as separate work for lists too long for the single-block scan
__global__ void k_check_counts(const int* num_neigh, int N, const int* first_neigh, int num_local_nodes, long num_edges,
                               long num_local_edges, int* status)
{
    int bad = 0;
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < N; i += (long)gridDim.x * blockDim.x) bad |= num_neigh[i] < 0;
    if (blockIdx.x == 0 && threadIdx.x == 0)
        bad |= (first_neigh[N] != (int)num_edges) | (first_neigh[num_local_nodes] != (int)num_local_edges);
    if (bad) atomicOr(status, 1);
}
// placement of entries that know their place inside the bucket: no atomics
__global__ void k_place_ranked(const int* key, const int* rank, long n, int rows, const int* start, int* list)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int j = key[i];
        if (j >= 0 && j < rows) list[start[j] + rank[i]] = (int)i;
    }
}
}  // namespace

hipError_t launch_node_lists_count(const int* num_neigh, int N, int* first_neigh, int* order, const int* node_types, int T,
                                   int* tstart, int* perm, const int* key, long n, int rows, int* count, int* rank,
                                   const InputChecks& chk, hipStream_t s)
{
    if (N <= 0 || N > 64 * SCAN_BLOCK || T <= 0) return hipErrorInvalidValue;
    const long work = chk.status ? std::max(n, chk.num_edges) : n;
    const unsigned nb = 3 + (unsigned)std::max<long>(1, std::min<long>((work + SCAN_BLOCK - 1) / SCAN_BLOCK, 2048));
    hipLaunchKernelGGL(k_node_lists_count, dim3(nb), dim3(SCAN_BLOCK), 2 * T * sizeof(int), s, num_neigh, N, first_neigh,
                       order, node_types, T, tstart, perm, key, n, rows, count, rank, chk);
    return hipGetLastError();
}
hipError_t launch_check_counts(const int* num_neigh, int N, const int* first_neigh, int num_local_nodes, long num_edges,
                               long num_local_edges, int* status, hipStream_t s)
{
    if (N > 0)
        hipLaunchKernelGGL(k_check_counts, dim3(std::min<unsigned>(nblk(N, 256), 1024u)), dim3(256), 0, s, num_neigh, N,
                           first_neigh, num_local_nodes, num_edges, num_local_edges, status);
    return hipGetLastError();
}

hipError_t launch_node_lists(const int* num_neigh, int N, int* first_neigh, int* order, const int* node_types, int T,
                             int* tstart, int* perm, int* zero_p, long zero_n, hipStream_t s)
{
    if (N <= 0 || N > 64 * SCAN_BLOCK || T <= 0) return hipErrorInvalidValue;
    hipLaunchKernelGGL(k_node_lists, dim3(1), dim3(SCAN_BLOCK), 2 * T * sizeof(int), s, num_neigh, N, first_neigh, order,
                       node_types, T, tstart, perm, zero_p, zero_n);
    return hipGetLastError();
}

hipError_t launch_scan_exclusive(const int* in, int* out, int n, int* block_sums, hipStream_t s)
{
    if (n <= 64 * SCAN_BLOCK) {
        hipLaunchKernelGGL(k_scan_single, dim3(1), dim3(SCAN_BLOCK), 0, s, in, out, n);
        return hipGetLastError();
    }
    const int nb = (n + SCAN_BLOCK - 1) / SCAN_BLOCK;
    hipLaunchKernelGGL(k_scan_tiles, dim3(nb), dim3(SCAN_BLOCK), 0, s, in, out, n, block_sums);
    hipLaunchKernelGGL(k_scan_sums, dim3(1), dim3(SCAN_BLOCK), 0, s, block_sums, nb, out, n);
    hipLaunchKernelGGL(k_scan_add, dim3(nb), dim3(SCAN_BLOCK), 0, s, out, n, block_sums);
    return hipGetLastError();
}

hipError_t launch_sender_lists(const int* gather, int E, int rows, int* count, int* sstart, int* cursor,
                               int* slist, int* block_sums, int counters_are_zero, const int* rank, hipStream_t s,
                               const InputGuard& guard)
{
    if (rows <= 0) return hipSuccess;
    const bool counted = counters_are_zero == 2;   // the histogram came with the node lists
    if (counters_are_zero) {
        // cleared by the previous build (or by k_node_lists)
    } else if (cursor == count + rows) {
        hipLaunchKernelGGL(k_fill<int>, dim3(nblk(2L * rows, 256)), dim3(256), 0, s, count, 2L * rows, 0);
    } else {
        hipLaunchKernelGGL(k_fill<int>, dim3(nblk(rows, 256)), dim3(256), 0, s, count, (long)rows, 0);
        hipLaunchKernelGGL(k_fill<int>, dim3(nblk(rows, 256)), dim3(256), 0, s, cursor, (long)rows, 0);
    }
    if (E > 0 && !counted) hipLaunchKernelGGL(k_count, dim3(nblk(E, 256)), dim3(256), 0, s, gather, (long)E, rows, count);
    hipError_t err = launch_scan_exclusive(count, sstart, rows, block_sums, s);
    if (err != hipSuccess) return err;
    if (E > 0) {
        if (counted && rank)
            hipLaunchKernelGGL(k_place_ranked, dim3(nblk(E, 256)), dim3(256), 0, s, gather, rank, (long)E, rows, sstart, slist);
        else
            hipLaunchKernelGGL(k_place, dim3(nblk(E, 256)), dim3(256), 0, s, gather, (long)E, rows, sstart, cursor, slist);
    }
    // the guard's bookkeeping rides on this launch, so it also runs for an edge list that claims to be empty
    if (E > 0 || guard.status)
        hipLaunchKernelGGL(k_sort_buckets, dim3(rows), dim3(64), 0, s, sstart, rows, slist, count, cursor, guard);
    return hipGetLastError();
}

hipError_t launch_type_groups(const int* node_types, int N, int T, int* tcount, int* tstart, int* cursor,
                              int* perm, int* block_sums, hipStream_t s)
{
    (void)tcount; (void)cursor; (void)block_sums;
    if (T <= 0) return hipSuccess;
    // order inside a species group is left as placed: every output row of the products
    // that use this grouping is computed independently of its tile mates
    hipLaunchKernelGGL(k_type_groups, dim3(1), dim3(1024), 2 * T * sizeof(int), s, node_types, N, T, tstart, perm);
    return hipGetLastError();
}

hipError_t launch_degree_order(int N, const int* first_neigh, int* order, hipStream_t s)
{
    if (N > 0) hipLaunchKernelGGL(k_degree_order, dim3(1), dim3(1024), 0, s, N, first_neigh, order);
    return hipGetLastError();
}

hipError_t launch_check_range(const int* v, long n, int limit, int* flags, hipStream_t s)
{
    if (n > 0) hipLaunchKernelGGL(k_check_range, dim3(nblk(n, 256)), dim3(256), 0, s, v, n, limit, flags);
    return hipGetLastError();
}
hipError_t launch_check_r(const double* r, long n, double r_cut, int* flags, hipStream_t s)
{
    if (n > 0) hipLaunchKernelGGL(k_check_r, dim3(nblk(n, 256)), dim3(256), 0, s, r, n, r_cut, flags);
    return hipGetLastError();
}
template <typename T>
hipError_t launch_fill(T* p, long n, T v, hipStream_t s)
{
    if (n > 0) hipLaunchKernelGGL(k_fill<T>, dim3(nblk(n, 256)), dim3(256), 0, s, p, n, v);
    return hipGetLastError();
}
template hipError_t launch_fill<double>(double*, long, double, hipStream_t);
template hipError_t launch_fill<float>(float*, long, float, hipStream_t);
template hipError_t launch_fill<int>(int*, long, int, hipStream_t);
template <typename TS, typename TD>
hipError_t launch_convert(const TS* src, TD* dst, long n, hipStream_t s)
{
    if (n > 0) hipLaunchKernelGGL((k_convert<TS, TD>), dim3(nblk(n, 256)), dim3(256), 0, s, src, dst, n);
    return hipGetLastError();
}
template hipError_t launch_convert<double, float>(const double*, float*, long, hipStream_t);
template hipError_t launch_convert<float, double>(const float*, double*, long, hipStream_t);
template hipError_t launch_convert<double, double>(const double*, double*, long, hipStream_t);
template hipError_t launch_convert<float, float>(const float*, float*, long, hipStream_t);

// ===========================================================================
// Symmetric contraction.  Atoms are grouped by species (list preparation); a
// thread owns one channel of two atoms of the same species, so every coefficient
// it loads (coalesced over channels, [species][monomial][K]) serves two
// evaluations.  The monomial indices come from the model file: the same for
// every lane, but not compile-time, so the 16 variables of each atom live in an
// LDS column ([17][block], slot 16 = the constant 1) that is only ever read in
// the loops.  The polynomial is walked once per variable v: the entries of list
// v give dP/dx_v = sum w x_fa x_fb in a register, written straight to M_grad;
// the monomials that start with v come first in the list, and
// P = sum_v x_v * (their partial sum).
namespace {
constexpr int POLY_BLOCK = 128;
// Atoms per thread: as many as fill one 16-byte LDS word, so that one ds_read_b128 brings a variable of
// all of them and every loaded coefficient serves them all.  (Twice as many was measured slower: fewer
// blocks than the chip holds at once.)
template <typename F> constexpr int poly_nb() { return 16 / (int)sizeof(F); }
typedef int __attribute__((address_space(4))) ConstInt;
template <typename F, int N>
struct alignas(16) PolyVec {
    F v[N];
};

// POLY_VG groups of POLY_BLOCK threads share the variables of a block in LDS; group g walks the lists of
// the variables v = g, g + POLY_VG, ...  A block is latency bound (every list entry needs a coefficient
// from L2), so spreading the 16 lists of an atom group over four times as many wavefronts shortens the
// kernel by nearly that factor.
constexpr int POLY_VG = POLY_GROUPS;
static_assert(16 % POLY_VG == 0 && POLY_BLOCK % 64 == 0 && POLY_SPARE_CHUNKS >= 2, "list layout and the kernel's walk must agree");

// Threads of a block: POLY_VG variable groups of PB threads each; thread `tid` of a group owns channel tid % CB of
// atom group tid / CB (AG atom groups of poly_nb atoms per block, PB = AG * CB rounded up to whole wavefronts).
// With K = 96 two atom groups fill three wavefronts exactly, where one group alone would leave a third of two
// wavefronts without a channel.
struct PolyShape {
    int CB, AG, PB;   // channels per block, atom groups per block, threads per variable group
};
static PolyShape poly_shape(int K, long atom_groups)
{
    PolyShape sh;
    sh.CB = K <= POLY_BLOCK ? K : POLY_BLOCK;
    sh.AG = 1;
    double best = 1e30;   // idle lanes per used lane; ties keep the smaller block
    for (int a = 1; a <= 4; a *= 2) {
        const int used = a * sh.CB, pb = (used + 63) / 64 * 64;
        if (a > 1 && pb > 192) break;
        if (a > 1 && atom_groups / a < 2 * 256) break;   // fewer than two blocks per CU: the lanes gained do not pay
        const double waste = (double)(pb - used) / used;
        if (waste < best - 1e-12) { best = waste; sh.AG = a; }
    }
    sh.PB = (sh.AG * sh.CB + 63) / 64 * 64;
    return sh;
}

template <typename F, int PB>
__global__ __launch_bounds__(PB * POLY_VG) void k_poly(const PolyParams<F> a, const PolyShape sh)
{
    constexpr int NB = poly_nb<F>();
    extern __shared__ __align__(16) unsigned char poly_smem[];
    PolyVec<F, NB>* Xs = reinterpret_cast<PolyVec<F, NB>*>(poly_smem);          // [17][PB]
    PolyVec<F, NB>* fsum = Xs + 17 * PB;                                         // [POLY_VG][PB]
    auto X = [&](int q) { return Xs + q * PB; };
    // the group index is the same for a whole wavefront: as a scalar it keeps the walk through the lists
    // (indices, chunk counts, coefficient rows) in scalar registers and scalar loads
    const int tid = threadIdx.x % PB, vg = __builtin_amdgcn_readfirstlane(threadIdx.x / PB);
    const int ag = tid / sh.CB, kloc = tid - ag * sh.CB;
    const bool tlive = ag < sh.AG;
    constexpr int VPG = 16 / POLY_VG;   // variables per group
    // species segment and atom groups of this block row
    const int kblocks = (a.K + sh.CB - 1) / sh.CB;
    int type = -1, sg = blockIdx.x / kblocks, seg0 = 0, seg_n = 0;
    for (int t = 0; t < a.T; ++t) {
        const int n_t = a.tstart[t + 1] - a.tstart[t];
        const int sgroups = ((n_t + NB - 1) / NB + sh.AG - 1) / sh.AG;
        if (sg < sgroups) { type = t; seg0 = a.tstart[t]; seg_n = n_t; break; }
        sg -= sgroups;
    }
    if (type < 0) return;
    const int grp = sg * sh.AG + (tlive ? ag : 0);
    const int k = (blockIdx.x % kblocks) * sh.CB + kloc;
    const bool klive = tlive && k < a.K;
    const unsigned kk = klive ? k : a.K - 1;
    int node[NB];
    bool nlive[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const int j = grp * NB + b;
        nlive[b] = tlive && j < seg_n;
        node[b] = a.perm[seg0 + (j < seg_n ? j : seg_n - 1)];
    }
    for (int q = vg; q < 17; q += POLY_VG) {
        PolyVec<F, NB> x;
#pragma unroll
        for (int b = 0; b < NB; ++b) x.v[b] = q < 16 ? a.A[((size_t)node[b] * 16 + q) * a.K + kk] : F(1);
        X(q)[tid] = x;
    }
    __syncthreads();
    for (int pl = 0; pl < a.NP; ++pl) {
        // the lists are read-only model data, the same for every lane: through the constant address space
        // they are fetched by scalar loads
        const ConstInt* pki = (const ConstInt*)a.packed[pl];
        auto pk = [&](int ch) { return make_int4(pki[4 * ch], pki[4 * ch + 1], pki[4 * ch + 2], pki[4 * ch + 3]); };
        const ConstInt* nch = (const ConstInt*)a.chunks[pl];
        // scalar base in the global address space; the lane adds kk
        typedef const F __attribute__((address_space(1))) GlobalF;
        GlobalF* coef = (GlobalF*)a.coef[pl] + (size_t)type * (a.num_entries[pl] + 1) * a.K;
        F f[NB], g[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) f[b] = g[b] = F(0);
        // this group's chunks are contiguous and start at c
        int c = 0;
        for (int q = 0; q < 2 * VPG * vg; ++q) c += nch[q];
        auto weights = [&](const int4& e, F (&w)[4]) {
            const int e4[4] = {e.x, e.y, e.z, e.w};
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = (coef + (size_t)(e4[q] & 0xffff) * a.K)[kk];
        };
        // indices two chunks ahead and coefficients one chunk ahead of the arithmetic, across the variables
        // of the group; the list ends with spare chunks of padding entries, so nothing here depends on where
        // the group's range stops
        int4 cur = pk(c), nxt = pk(c + 1);
        F w[4];
        weights(cur, w);
        // The gradients of the group's variables stay in registers until all lists are walked: a store between
        // the lists would sit in front of the next coefficient loads, whose wait would then wait for it too.
        F gs[VPG][NB];
#pragma unroll
        for (int t = 0; t < VPG; ++t) {
            const int v = vg + POLY_VG * t;
            const int n0 = nch[2 * (VPG * vg + t)], n1 = nch[2 * (VPG * vg + t) + 1];
#pragma unroll
            for (int b = 0; b < NB; ++b) g[b] = F(0);
            for (int i = 0; i < n0 + n1; ++i, ++c) {
                F wn[4];
                weights(nxt, wn);
                const int4 nn = pk(c + 2);
                const int e4[4] = {cur.x, cur.y, cur.z, cur.w};
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int ia = (e4[q] >> 16) & 0xff, ib = (e4[q] >> 24) & 0xff;
                    const PolyVec<F, NB> xa = X(ia)[tid], xb = X(ib)[tid];
#pragma unroll
                    for (int b = 0; b < NB; ++b) g[b] += w[q] * (xa.v[b] * xb.v[b]);
                }
                cur = nxt; nxt = nn;
#pragma unroll
                for (int q = 0; q < 4; ++q) w[q] = wn[q];
                if (i + 1 == n0) {
                    // the monomials that start with v are done: their sum times x_v is v's share of P
                    const PolyVec<F, NB> xv = X(v)[tid];
#pragma unroll
                    for (int b = 0; b < NB; ++b) f[b] += xv.v[b] * g[b];
                }
            }
#pragma unroll
            for (int b = 0; b < NB; ++b) gs[t][b] = g[b];
        }
#pragma unroll
        for (int t = 0; t < VPG; ++t)
#pragma unroll
            for (int b = 0; b < NB; ++b)
                if (klive && nlive[b])
                    a.M_grad[(((size_t)node[b] * a.NP + pl) * 16 + vg + POLY_VG * t) * a.K + k] = gs[t][b];
        // P = sum of the groups' shares, added in group order
        {
            PolyVec<F, NB> fv;
#pragma unroll
            for (int b = 0; b < NB; ++b) fv.v[b] = f[b];
            fsum[vg * PB + tid] = fv;
        }
        __syncthreads();
        if (vg == 0) {
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                F t = F(0);
#pragma unroll
                for (int g2 = 0; g2 < POLY_VG; ++g2) t += fsum[g2 * PB + tid].v[b];
                if (klive && nlive[b]) a.M[((size_t)node[b] * a.NP + pl) * a.K + k] = t;
            }
        }
        __syncthreads();
    }
}


template <typename F, int V>
struct alignas(sizeof(F) * V > 16 ? 16 : sizeof(F) * V) RevVec {
    F v[V];
};
// four consecutive channels per thread when K allows 16/32-byte accesses (V = 4), else one
template <typename F, int V>
__global__ void k_poly_reverse(long total_v, int NP, int K, const F* M_grad, const F* M_adj, F* A_adj)
{
    const long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;  // over [N][16][K / V]
    if (idx >= total_v) return;
    const int KV = K / V;
    const int kq = (int)(idx % KV) * V;
    const long t = idx / KV;
    const int lm = (int)(t % 16);
    const long i = t / 16;
    RevVec<F, V> s;
#pragma unroll
    for (int j = 0; j < V; ++j) s.v[j] = F(0);
    for (int p = 0; p < NP; ++p) {
        const RevVec<F, V> g = *reinterpret_cast<const RevVec<F, V>*>(M_grad + ((i * NP + p) * 16 + lm) * K + kq);
        const RevVec<F, V> m = *reinterpret_cast<const RevVec<F, V>*>(M_adj + (i * NP + p) * K + kq);
#pragma unroll
        for (int j = 0; j < V; ++j) s.v[j] += g.v[j] * m.v[j];
    }
    *reinterpret_cast<RevVec<F, V>*>(A_adj + (i * 16 + lm) * K + kq) = s;
}
}  // namespace

template <typename F>
hipError_t launch_poly(const PolyParams<F>& p, hipStream_t s)
{
    if (p.num_nodes <= 0) return hipSuccess;
    if (p.table_slabs) return launch_poly_spec<F>(p, s);   // standard product basis (smx_kernels_poly.hip)
    if (p.mode != 0) return hipErrorInvalidValue;   // the general kernel has the one mode
    const PolyShape sh = poly_shape(p.K, (p.num_nodes + poly_nb<F>() - 1) / poly_nb<F>());
    const int kblocks = (p.K + sh.CB - 1) / sh.CB;
    const int per_block = poly_nb<F>() * sh.AG;
    const unsigned sgroups = (unsigned)((p.num_nodes + per_block - 1) / per_block + p.T);
    const size_t lds = (size_t)(17 + POLY_VG) * sh.PB * 16;
    auto go = [&](auto pbc) -> hipError_t {
        constexpr int PB = decltype(pbc)::value;
        static bool attr_done = false;   // per instantiation
        if (!attr_done) {
            hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_poly<F, PB>), hipFuncAttributeMaxDynamicSharedMemorySize, 96 * 1024);
            if (err != hipSuccess) return err;
            attr_done = true;
        }
        hipLaunchKernelGGL((k_poly<F, PB>), dim3(sgroups * kblocks), dim3(PB * POLY_VG), lds, s, p, sh);
        return hipGetLastError();
    };
    switch (sh.PB) {
    case 64: return go(std::integral_constant<int, 64>{});
    case 128: return go(std::integral_constant<int, 128>{});
    case 192: return go(std::integral_constant<int, 192>{});
    default: return hipErrorInvalidValue;
    }
}
template hipError_t launch_poly<double>(const PolyParams<double>&, hipStream_t);
template hipError_t launch_poly<float>(const PolyParams<float>&, hipStream_t);

template <typename F>
hipError_t launch_poly_reverse(int N, int NP, int K, const F* M_grad, const F* M_adj, F* A_adj, hipStream_t s)
{
    if (N <= 0) return hipSuccess;
    if (K % 4 == 0) {
        const long total = (long)N * 16 * (K / 4);
        hipLaunchKernelGGL((k_poly_reverse<F, 4>), dim3(nblk(total, 256)), dim3(256), 0, s, total, NP, K, M_grad, M_adj, A_adj);
    } else {
        const long total = (long)N * 16 * K;
        hipLaunchKernelGGL((k_poly_reverse<F, 1>), dim3(nblk(total, 256)), dim3(256), 0, s, total, NP, K, M_grad, M_adj, A_adj);
    }
    return hipGetLastError();
}
template hipError_t launch_poly_reverse<double>(int, int, int, const double*, const double*, double*, hipStream_t);
template hipError_t launch_poly_reverse<float>(int, int, int, const float*, const float*, float*, hipStream_t);

// ===========================================================================
// Readout tail
// The whole readout tail in one launch (mace.cpp:876-903, multilayer_perceptron.cpp:76-150): the K -> 16 -> 1
// network on H2 with its gradient (H2_adj), the linear readout of H1's scalar block, the atomic energy, and the
// seed of H1_adj (readout weights in the scalar block of the first N rows, zero elsewhere).  A block serves 16
// nodes; thread (node, hidden unit) forms one hidden activation with the K products taken in ascending order.
namespace {
template <typename F>
__global__ __launch_bounds__(256) void k_readout_fused(int N, int rows, int K, int num_LM, const int* node_types,
                                                       const double* E0, const double* w1, const double* W1,
                                                       const double* w2, double scale, const F* H1, const double* H2,
                                                       double* H2_adj, F* H1_adj, double* node_energies,
                                                       int zero_energies, double* energies_copy, const int* guard,
                                                       int* guard_clear, double* guard_forces, long guard_forces_n)
{
    extern __shared__ double rsm[];
    // every reader of the check word has run (the sender lists come before the readout): clean for the next evaluation
    if (guard_clear && blockIdx.x == 0 && threadIdx.x == 0) *guard_clear = 0;
    if (guard && *guard) {
        // unchecked species indices: no table lookup, the energies say so; so do the edge forces, which the
        // adjoint kernels of this evaluation will not touch (they see no edges)
        const int i = blockIdx.x * 16 + (threadIdx.x >> 4);
        if ((threadIdx.x & 15) == 0 && i < N) {
            node_energies[i] = __builtin_nan("");
            if (energies_copy) energies_copy[i] = __builtin_nan("");
        }
        for (long t = (long)blockIdx.x * 256 + threadIdx.x; t < guard_forces_n; t += (long)gridDim.x * 256)
            guard_forces[t] = __builtin_nan("");
        return;
    }
    const int ldw = K + 1;                 // rows of W1 start two banks apart
    double* W = rsm;                       // [16][K + 1]
    double* hg = W + 16 * ldw;             // [16 nodes][16]
    double* X = hg + 256;                  // [16 nodes][K]: the block's rows of H2
    for (int t = threadIdx.x; t < 16 * K; t += 256) {
        W[(t / K) * ldw + t % K] = W1[t];
        const size_t src = (size_t)blockIdx.x * 16 * K + t;
        X[t] = src < (size_t)N * K ? H2[src] : 0.0;
    }
    __syncthreads();
    const int n = threadIdx.x >> 4, h = threadIdx.x & 15;
    const int i = blockIdx.x * 16 + n;
    double e = 0.0, g = 0.0;
    if (i < N) {
        const double* h2 = X + n * K;
        double s = 0.0;
#pragma unroll 8
        for (int k = 0; k < K; ++k) s += W[h * ldw + k] * h2[k];
        // multilayer_perceptron.cpp:107-113: scaled SiLU and its derivative
        const double sig = 1.0 / (1.0 + exp(-s));
        e = w2[h] * (scale * s * sig);
        g = w2[h] * (scale * sig + scale * s * sig * (1 - sig));
        const F* Hs = H1 + (size_t)i * num_LM * K;
        for (int k = h; k < K; k += 16) e += w1[k] * (double)Hs[k];
    }
#pragma unroll
    for (int off = 8; off >= 1; off >>= 1) e += __shfl_xor(e, off, 64);
    hg[threadIdx.x] = g;
    if (h == 0 && i < N) {
        const double en = (zero_energies ? 0.0 : node_energies[i]) + E0[node_types[i]] + e;
        node_energies[i] = en;
        if (energies_copy) energies_copy[i] = en;
    }
    __syncthreads();
    for (int t = threadIdx.x; t < 16 * K; t += 256) {
        const int n2 = t / K, k = t - n2 * K;
        const int i2 = blockIdx.x * 16 + n2;
        if (i2 < N) {
            double s = 0.0;
#pragma unroll
            for (int q = 0; q < 16; ++q) s += hg[n2 * 16 + q] * W[q * ldw + k];
            H2_adj[(size_t)i2 * K + k] = s;
        }
    }
    const int width = num_LM * K;
    for (int t = threadIdx.x; t < 16 * width; t += 256) {
        const int n2 = t / width, c = t - n2 * width;
        const int row = blockIdx.x * 16 + n2;
        if (row < rows) H1_adj[(size_t)row * width + c] = (c < K && row < N) ? (F)w1[c] : F(0);
    }
}
}  // namespace

// ---------------------------------------------------------------------------
// H2, the readout tail above and reverse_H2 in one launch (mace.cpp:820-903).  All three work on one atom's
// rows only.  A block takes 16 atoms of one species (species groups of the list preparation) through:
//   H2 = H1[l=0] . W_H1[type] + M1 . W_M1 on the matrix cores (operands from LDS, weights straight from
//   L2 in the operand layout: a 16-lane group reads 16 consecutive columns of one weight row),
//   the K -> 16 -> 1 network with its gradient H2_adj, energies, the seed of H1_adj,
//   H1_adj[l=0] += H2_adj . W_H1[type]^T and M1_adj = H2_adj . W_M1^T (a lane reads 32 consecutive bytes of
//   its weight row; k is permuted inside groups of 16 on both operands).
// Sums over k run in one fixed order per output element, independent of the atom's tile mates.
namespace {
typedef double f64x4 __attribute__((ext_vector_type(4)));
constexpr int TAIL_BLOCK = 512;   // eight wavefronts: wavefront w owns column tile w of both products
template <typename F, int KT>
__global__ __launch_bounds__(TAIL_BLOCK) void k_tail_fused(const TailParams<F> p)
{
    extern __shared__ double tsm[];
    constexpr int K = 16 * KT, ld = K + 1;   // padded rows: a column read by 16 rows hits 16 banks
    double* W1s = tsm;                       // [16][ld]
    double* hg = W1s + 16 * ld;              // [16 atoms][16 hidden]
    double* XA = hg + 256;                   // [16][ld] H1[l=0] rows
    double* XB = XA + 16 * ld;               // [16][ld] M1 rows
    double* XH = XB + 16 * ld;               // [16][ld] H2 rows
    double* XY = XH + 16 * ld;               // [16][ld] H2_adj rows
    __shared__ int node_s[16];
    const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int width = p.num_LM * K;
    // every reader of the check word has run (the sender lists come before the readout): clean for the next evaluation
    if (p.guard_clear && blockIdx.x == 0 && tid == 0) *p.guard_clear = 0;
    if (p.guard && *p.guard) {
        // the inputs of this evaluation failed their checks and the species groups are empty: the energies say so
        const int i = blockIdx.x * 16 + tid;
        if (tid < 16 && i < p.N) {
            p.node_energies[i] = __builtin_nan("");
            if (p.energies_copy) p.energies_copy[i] = __builtin_nan("");
        }
        // ... and so do the edge forces, which the adjoint kernels will not touch (they see no edges)
        for (long t = (long)blockIdx.x * TAIL_BLOCK + tid; t < p.guard_forces_n; t += (long)gridDim.x * TAIL_BLOCK)
            p.guard_forces[t] = __builtin_nan("");
        return;
    }
    // rows beyond the atoms (ghost rows of H1_adj) are cleared by all blocks together
    {
        const long ghost = (long)(p.rows - p.N) * width;
        for (long t = (long)blockIdx.x * TAIL_BLOCK + tid; t < ghost; t += (long)gridDim.x * TAIL_BLOCK)
            p.H1_adj[(size_t)p.N * width + t] = F(0);
    }
    // species segment and tile of this block
    int type = -1, tile = blockIdx.x, seg0 = 0, seg_n = 0;
    for (int t = 0; t < p.T; ++t) {
        const int n_t = p.tstart[t + 1] - p.tstart[t];
        const int tiles = (n_t + 15) / 16;
        if (tile < tiles) { type = t; seg0 = p.tstart[t]; seg_n = n_t; break; }
        tile -= tiles;
    }
    if (type < 0) return;
    const int r = lane & 15, g = lane >> 4;
    const double* WH = p.W_H1 + (size_t)type * K * K;
    const bool owner = wave < KT;            // this wavefront owns column tile `wave`
    // the weights of the first product pair are requested before anything else: they do not depend on the atoms
    double b1[K / 4], b2[K / 4];
    if (owner) {
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
            b1[q] = WH[(size_t)(4 * q + g) * K + wave * 16 + r];
            b2[q] = p.W_M1[(size_t)(4 * q + g) * K + wave * 16 + r];
        }
    }
    if (tid < 16) node_s[tid] = tile * 16 + tid < seg_n ? p.perm[seg0 + tile * 16 + tid] : -1;
    __syncthreads();
    for (int t = tid; t < 16 * K; t += TAIL_BLOCK) {
        const int rr = t / K, k = t - rr * K;
        W1s[rr * ld + k] = p.W1[t];
        const int nd = node_s[rr];
        XA[rr * ld + k] = nd >= 0 ? (double)p.H1[(size_t)nd * width + k] : 0.0;
        XB[rr * ld + k] = nd >= 0 ? (double)p.M1[(size_t)nd * K + k] : 0.0;
    }
    __syncthreads();
    // ---- H2 tile
    f64x4 w1v[KT], w2v[KT];                   // weights of the transposed products, requested early as well
    if (owner) {
        f64x4 acc1 = {0, 0, 0, 0}, acc2 = {0, 0, 0, 0};
#pragma unroll
        for (int q = 0; q < K / 4; ++q) {
            acc1 = __builtin_amdgcn_mfma_f64_16x16x4f64(XA[r * ld + 4 * q + g], b1[q], acc1, 0, 0, 0);
            acc2 = __builtin_amdgcn_mfma_f64_16x16x4f64(XB[r * ld + 4 * q + g], b2[q], acc2, 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < KT; ++j) {
            w1v[j] = *reinterpret_cast<const f64x4*>(WH + (size_t)(wave * 16 + r) * K + 16 * j + 4 * g);
            w2v[j] = *reinterpret_cast<const f64x4*>(p.W_M1 + (size_t)(wave * 16 + r) * K + 16 * j + 4 * g);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int row = 4 * q + g, col = wave * 16 + r;
            const double v = acc1[q] + acc2[q];
            XH[row * ld + col] = v;
            const int nd = node_s[row];
            if (nd >= 0) p.H2[(size_t)nd * K + col] = v;
        }
    }
    __syncthreads();
    // ---- readout network, energies (thread = atom n, hidden unit h)
    if (tid < 256) {
        const int n = tid >> 4, h = tid & 15;
        const int i = node_s[n];
        double e = 0.0, gr = 0.0;
        if (i >= 0) {
            const double* h2 = XH + n * ld;
            double sdot = 0.0;
#pragma unroll 8
            for (int k = 0; k < K; ++k) sdot += W1s[h * ld + k] * h2[k];
            // multilayer_perceptron.cpp:107-113: scaled SiLU and its derivative
            const double sig = 1.0 / (1.0 + exp(-sdot));
            e = p.w2[h] * (p.scale * sdot * sig);
            gr = p.w2[h] * (p.scale * sig + p.scale * sdot * sig * (1 - sig));
            for (int k = h; k < K; k += 16) e += p.w1[k] * XA[n * ld + k];
        }
#pragma unroll
        for (int off = 8; off >= 1; off >>= 1) e += __shfl_xor(e, off, 64);
        hg[tid] = gr;
        if (h == 0 && i >= 0) {
            const double en = (p.zero_energies ? 0.0 : p.node_energies[i]) + p.E0[type] + e;
            p.node_energies[i] = en;
            if (p.energies_copy) p.energies_copy[i] = en;
        }
    }
    __syncthreads();
    // ---- H2_adj tile
    for (int t = tid; t < 16 * K; t += TAIL_BLOCK) {
        const int n2 = t / K, k = t - n2 * K;
        double sum = 0.0;
#pragma unroll
        for (int q = 0; q < 16; ++q) sum += hg[n2 * 16 + q] * W1s[q * ld + k];
        XY[n2 * ld + k] = sum;
        const int nd = node_s[n2];
        if (nd >= 0) p.H2_adj[(size_t)nd * K + k] = sum;
    }
    __syncthreads();
    // ---- H1_adj[l=0] = w1 + H2_adj . W_H1^T, M1_adj = H2_adj . W_M1^T
    if (owner) {
        f64x4 acc1 = {0, 0, 0, 0}, acc2 = {0, 0, 0, 0};
        const double* a = XY + r * ld + 4 * g;
#pragma unroll
        for (int j = 0; j < KT; ++j) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                acc1 = __builtin_amdgcn_mfma_f64_16x16x4f64(a[16 * j + t], w1v[j][t], acc1, 0, 0, 0);
                acc2 = __builtin_amdgcn_mfma_f64_16x16x4f64(a[16 * j + t], w2v[j][t], acc2, 0, 0, 0);
            }
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int nd = node_s[4 * q + g], col = wave * 16 + r;
            if (nd >= 0) {
                p.H1_adj[(size_t)nd * width + col] = (F)((double)(F)p.w1[col] + acc1[q]);
                p.M1_adj[(size_t)nd * K + col] = (F)acc2[q];
            }
        }
    }
    // the other blocks of H1_adj start at zero
    for (int t = tid; t < 16 * (width - K); t += TAIL_BLOCK) {
        const int n2 = t / (width - K), c = K + t - n2 * (width - K);
        const int nd = node_s[n2];
        if (nd >= 0) p.H1_adj[(size_t)nd * width + c] = F(0);
    }
}
}  // namespace

template <typename F>
size_t tail_fused_lds(int K) { return ((size_t)5 * 16 * (K + 1) + 256) * sizeof(double); }
bool tail_fused_ok(int K) { return K == 32 || K == 48 || K == 64 || K == 96 || K == 128; }

template <typename F, int KT>
static hipError_t launch_tail_fused_t(const TailParams<F>& p, hipStream_t s)
{
    const size_t lds = tail_fused_lds<F>(p.K);
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_tail_fused<F, KT>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    const unsigned blocks = (unsigned)((p.N + 15) / 16 + p.T);
    hipLaunchKernelGGL((k_tail_fused<F, KT>), dim3(blocks), dim3(TAIL_BLOCK), lds, s, p);
    return hipGetLastError();
}
template <typename F>
hipError_t launch_tail_fused(const TailParams<F>& p, hipStream_t s)
{
    if (p.rows < p.N || !tail_fused_ok(p.K) || p.T <= 0) return hipErrorInvalidValue;
    if (p.rows <= 0) return hipSuccess;
    switch (p.K / 16) {
    case 2: return launch_tail_fused_t<F, 2>(p, s);
    case 3: return launch_tail_fused_t<F, 3>(p, s);
    case 4: return launch_tail_fused_t<F, 4>(p, s);
    case 6: return launch_tail_fused_t<F, 6>(p, s);
    default: return launch_tail_fused_t<F, 8>(p, s);
    }
}
template hipError_t launch_tail_fused<double>(const TailParams<double>&, hipStream_t);
template hipError_t launch_tail_fused<float>(const TailParams<float>&, hipStream_t);

template <typename F>
hipError_t launch_readout_fused(int N, int rows, int K, int num_LM, const int* node_types, const double* atomic_energies,
                                const double* w1, const double* W1, const double* w2, double scale, const F* H1,
                                const double* H2, double* H2_adj, F* H1_adj, double* node_energies, int zero_energies,
                                double* energies_copy, const int* guard, int* guard_clear, double* guard_forces,
                                long guard_forces_n, hipStream_t s)
{
    if (rows < N) return hipErrorInvalidValue;
    if (rows <= 0) return hipSuccess;
    const size_t lds = ((size_t)16 * (K + 1) + 256 + (size_t)16 * K) * sizeof(double);
    if (lds > 160 * 1024) return hipErrorInvalidValue;    // K beyond about 630 channels
    if (lds > 64 * 1024) {
        hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(k_readout_fused<F>),
                                             hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    hipLaunchKernelGGL(k_readout_fused<F>, dim3((rows + 15) / 16), dim3(256), lds, s, N, rows, K, num_LM, node_types,
                       atomic_energies, w1, W1, w2, scale, H1, H2, H2_adj, H1_adj, node_energies, zero_energies,
                       energies_copy, guard, guard_clear, guard_forces, guard_forces_n);
    return hipGetLastError();
}
template hipError_t launch_readout_fused<double>(int, int, int, int, const int*, const double*, const double*, const double*, const double*, double, const double*, const double*, double*, double*, double*, int, double*, const int*, int*, double*, long, hipStream_t);
template hipError_t launch_readout_fused<float>(int, int, int, int, const int*, const double*, const double*, const double*, const double*, double, const float*, const double*, double*, float*, double*, int, double*, const int*, int*, double*, long, hipStream_t);


// ===========================================================================
// Caller-side reductions: per-edge forces -> per-atom forces (each atom sums its
// own incoming and outgoing edges in ascending edge order: no atomics), virial.
namespace {
__global__ void k_force_scatter(int num_atoms, const int* recv_start, const int* recv_list, const int* send_start,
                                const int* send_list, const double* forces, double* atom_forces)
{
    const int a = blockIdx.x * blockDim.x + threadIdx.x;
    if (a >= num_atoms) return;
    double fx = 0, fy = 0, fz = 0;
    for (int t = send_start[a]; t < send_start[a + 1]; ++t) {
        const size_t e = send_list[t];
        fx += forces[3 * e]; fy += forces[3 * e + 1]; fz += forces[3 * e + 2];
    }
    for (int t = recv_start[a]; t < recv_start[a + 1]; ++t) {
        const size_t e = recv_list ? recv_list[t] : t;
        fx -= forces[3 * e]; fy -= forces[3 * e + 1]; fz -= forces[3 * e + 2];
    }
    atom_forces[3 * (size_t)a] = fx; atom_forces[3 * (size_t)a + 1] = fy; atom_forces[3 * (size_t)a + 2] = fz;
}
__global__ __launch_bounds__(256) void k_virial(long E, const double* xyz, const double* f, double* partial)
{
    __shared__ double red[6][256];
    double v[6] = {0, 0, 0, 0, 0, 0};
    // fixed assignment of edges to threads, fixed tree: deterministic
    for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < E; e += (long)gridDim.x * blockDim.x) {
        const double x = xyz[3 * e], y = xyz[3 * e + 1], z = xyz[3 * e + 2];
        const double fx = f[3 * e], fy = f[3 * e + 1], fz = f[3 * e + 2];
        v[0] += x * fx; v[1] += y * fy; v[2] += z * fz;
        v[3] += 0.5 * (x * fy + y * fx); v[4] += 0.5 * (x * fz + z * fx); v[5] += 0.5 * (y * fz + z * fy);
    }
    for (int q = 0; q < 6; ++q) red[q][threadIdx.x] = v[q];
    __syncthreads();
    for (int off = 128; off >= 1; off >>= 1) {
        if ((int)threadIdx.x < off)
            for (int q = 0; q < 6; ++q) red[q][threadIdx.x] += red[q][threadIdx.x + off];
        __syncthreads();
    }
    if (threadIdx.x < 6) partial[blockIdx.x * 6 + threadIdx.x] = red[threadIdx.x][0];
}
}  // namespace

hipError_t launch_force_scatter(int num_atoms, const int* recv_start, const int* recv_list, const int* send_start,
                                const int* send_list, const double* forces, double* atom_forces, hipStream_t s)
{
    if (num_atoms > 0)
        hipLaunchKernelGGL(k_force_scatter, dim3(nblk(num_atoms, 128)), dim3(128), 0, s, num_atoms, recv_start,
                           recv_list, send_start, send_list, forces, atom_forces);
    return hipGetLastError();
}
hipError_t launch_virial(long E, const double* xyz, const double* forces, double* partial, int nblocks, hipStream_t s)
{
    hipLaunchKernelGGL(k_virial, dim3(nblocks), dim3(256), 0, s, E, xyz, forces, partial);
    return hipGetLastError();
}

}  // namespace smx
