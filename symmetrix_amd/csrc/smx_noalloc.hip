// smx_reduce_forces_device_noalloc: the force / virial reduction of smx_reduce_forces_device for callers that
// cannot allocate (code under HIP graph capture, serving loops, harnesses that forbid hipMalloc).  Its working
// arrays -- the per-atom sender lists and the partial virial sums, which the allocating entry point keeps in
// growable buffers -- live in one file-scope device array of fixed size.  Every call on a GPU shares that GPU's
// copy of the array: calls that overlap on one GPU race.
#include <hip/hip_runtime.h>

#include <string>

#include "../../include/symmetrix_amd.h"
#include "smx_internal.hpp"
#include "smx_kernels.hpp"

namespace {

constexpr int kMaxAtoms = SMX_NOALLOC_MAX_ATOMS;
constexpr long kMaxEdges = SMX_NOALLOC_MAX_EDGES;
constexpr int kVirialBlocks = 64;

constexpr size_t align256(size_t n) { return (n + 255) / 256 * 256; }
// layout of the scratch array (byte offsets, every part 256-byte aligned)
constexpr size_t kOffFlag = 0;                                                          // int[64]
constexpr size_t kOffCount = kOffFlag + 256;                                            // int[2 * atoms]: counters, cursors
constexpr size_t kOffSendStart = kOffCount + align256(2 * (size_t)kMaxAtoms * sizeof(int));     // int[atoms + 1]
constexpr size_t kOffRecvStart = kOffSendStart + align256(((size_t)kMaxAtoms + 1) * sizeof(int)); // int[atoms + 1]
constexpr size_t kOffBlockSums = kOffRecvStart + align256(((size_t)kMaxAtoms + 1) * sizeof(int)); // int[atoms / 1024 + 2]
constexpr size_t kOffSendList = kOffBlockSums + align256(((size_t)kMaxAtoms / 1024 + 2) * sizeof(int)); // int[edges]
constexpr size_t kOffVirial = kOffSendList + align256((size_t)kMaxEdges * sizeof(int));  // double[64 * 6]
constexpr size_t kScratchBytes = kOffVirial + align256((size_t)kVirialBlocks * 6 * sizeof(double));

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// address of this device's copy of `scratch`, looked up once per device (the name itself is no device address
// in host code)
constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

// receiver block i is atom i: CSR offsets of the receivers, padded with the edge count for atoms beyond them
__global__ void k_pad_starts(const int* first_neigh, int num_receivers, int num_atoms, int* out)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i <= num_atoms) out[i] = first_neigh[i < num_receivers ? i : num_receivers];
}
// the partial sums in ascending block order, as the allocating entry point adds them on the host
__global__ void k_virial_finish(const double* partial, int nblocks, const int* flag, double* virial)
{
    const int q = threadIdx.x;
    if (q >= 6) return;
    double v = 0.0;
    for (int b = 0; b < nblocks; ++b) v += partial[(size_t)b * 6 + q];
    virial[q] = *flag ? __builtin_nan("") : v;
}
// an out-of-range sender index cannot be reported through a return code without a host synchronisation:
// the outputs are NaN instead
__global__ void k_poison_if_flag(const int* flag, double* out, long n)
{
    const long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n && *flag) out[i] = __builtin_nan("");
}

}  // namespace

namespace smx {

int noalloc_setup_current_device(std::string* err)
{
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) { if (err) *err = std::string("hipGetDevice: ") + hipGetErrorString(e); return SMX_EHIP; }
    if (dev < 0 || dev >= kMaxDevices) { if (err) *err = "device ordinal beyond the per-device table of the no-allocation entry point"; return SMX_EINVAL; }
    if (g_scratch_ptr[dev]) return SMX_OK;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
        if (err) *err = std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e);
        return SMX_EHIP;
    }
    g_scratch_ptr[dev] = static_cast<unsigned char*>(p);
    return SMX_OK;
}

}  // namespace smx

extern "C" int smx_reduce_forces_device_noalloc(smx_model* m, int num_atoms, const int* d_sender_atom,
                                                double* d_atom_forces, double* d_virial, void* stream)
{
    std::string err;
    smx::ForcesView v{};
    int rc = smx::engine_forces_view(m, &v, &err);
    if (rc != SMX_OK) { smx::set_last_error(err); return rc; }
    if (num_atoms <= 0 || !d_sender_atom || (!d_atom_forces && !d_virial)) {
        smx::set_last_error("smx_reduce_forces_device_noalloc: num_atoms must be positive, sender_atom and one output not null");
        return SMX_EINVAL;
    }
    if (num_atoms > kMaxAtoms || v.num_edges > kMaxEdges) {
        smx::set_last_error("smx_reduce_forces_device_noalloc: " + std::to_string(num_atoms) + " atoms / " +
                            std::to_string(v.num_edges) + " edges exceed the fixed scratch array (at most " +
                            std::to_string(kMaxAtoms) + " atoms and " + std::to_string(kMaxEdges) +
                            " edges); use smx_reduce_forces_device");
        return SMX_EINVAL;
    }
    if (num_atoms < v.num_receivers) {
        smx::set_last_error("num_atoms is smaller than the number of receivers");
        return SMX_EINVAL;
    }
    if (!v.node_forces || v.forces_len != 3 * v.num_edges) {
        smx::set_last_error("node_forces does not match the current edge list");
        return SMX_EINVAL;
    }
    rc = smx::noalloc_setup_current_device(&err);
    if (rc != SMX_OK) { smx::set_last_error(err); return rc; }
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev != v.device) {
        smx::set_last_error("smx_reduce_forces_device_noalloc: the current device (" + std::to_string(dev) +
                            ") is not the one the model lives on (" + std::to_string(v.device) + ")");
        return SMX_EINVAL;
    }
    unsigned char* base = g_scratch_ptr[dev];
    hipStream_t s = static_cast<hipStream_t>(stream);
    int* flag = reinterpret_cast<int*>(base + kOffFlag);
    int* count = reinterpret_cast<int*>(base + kOffCount);
    int* send_start = reinterpret_cast<int*>(base + kOffSendStart);
    int* recv_start = reinterpret_cast<int*>(base + kOffRecvStart);
    int* block_sums = reinterpret_cast<int*>(base + kOffBlockSums);
    int* send_list = reinterpret_cast<int*>(base + kOffSendList);
    double* partial = reinterpret_cast<double*>(base + kOffVirial);
    const long E = v.num_edges;
    hipError_t e = smx::launch_fill<int>(flag, 1, 0, s);
    if (e == hipSuccess) e = smx::launch_check_range(d_sender_atom, E, num_atoms, flag, s);
    if (e == hipSuccess && d_atom_forces) {
        // counters and cursors of the last call are cleared inside (a fill kernel, no memset node)
        e = smx::launch_sender_lists(d_sender_atom, (int)E, num_atoms, count, send_start, count + num_atoms, send_list,
                                     block_sums, 0, nullptr, s);
        if (e == hipSuccess) {
            hipLaunchKernelGGL(k_pad_starts, dim3((num_atoms + 256) / 256), dim3(256), 0, s, v.first_neigh, v.num_receivers,
                               num_atoms, recv_start);
            e = hipGetLastError();
        }
        if (e == hipSuccess) e = smx::launch_force_scatter(num_atoms, recv_start, nullptr, send_start, send_list, v.node_forces, d_atom_forces, s);
        if (e == hipSuccess) {
            const long n = 3L * num_atoms;
            hipLaunchKernelGGL(k_poison_if_flag, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, flag, d_atom_forces, n);
            e = hipGetLastError();
        }
    }
    if (e == hipSuccess && d_virial) {
        e = smx::launch_virial(E, v.xyz, v.node_forces, partial, kVirialBlocks, s);
        if (e == hipSuccess) {
            hipLaunchKernelGGL(k_virial_finish, dim3(1), dim3(64), 0, s, partial, kVirialBlocks, flag, d_virial);
            e = hipGetLastError();
        }
    }
    if (e != hipSuccess) {
        smx::set_last_error(std::string("smx_reduce_forces_device_noalloc: ") + hipGetErrorString(e));
        return SMX_EHIP;
    }
    return SMX_OK;
}
