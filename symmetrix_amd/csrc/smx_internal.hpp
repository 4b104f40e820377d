// Shared between the translation units that implement the C ABI (not part of it).
#pragma once

#include <string>

struct smx_model;

namespace smx {

// device arrays of the model's last evaluation that the caller-side reductions read
struct ForcesView {
    const double* node_forces;   // [num_edges][3]
    const double* xyz;           // [num_edges][3]
    const int* first_neigh;      // [num_receivers + 1]
    long num_edges, forces_len;
    int num_receivers;
    int device;                  // ordinal of the GPU that holds the model and these arrays
};
int engine_forces_view(smx_model* m, ForcesView* out, std::string* err);
void set_last_error(const std::string& msg);

// looks up this device's copy of the scratch array of the no-allocation entry point (once per device)
int noalloc_setup_current_device(std::string* err);

}  // namespace smx
