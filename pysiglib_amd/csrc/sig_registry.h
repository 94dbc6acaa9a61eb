// Host-side table of compiled tree-kernel instances and their launchers.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sigamd {

struct FwdParams {
    const void* inc;
    void* out;
    int64_t batch, L;
    int d;
    int64_t out_stride;
    int scalar;
    hipStream_t stream;
    int nseg;        // time segments per path; batch counts (path, segment) items
    int64_t lseg;    // increments per segment
    int* nonfinite = nullptr;   // device-visible flag set when a stored value is NaN or infinite (may be null)
    int from_points = 0;        // staged kernels of at most kPointFedMaxDim channels: inc is the plain path [batch][L + 1][d]
};
constexpr int kPointFedMaxDim = 16;

struct BwdParams {
    const void* inc;
    const void* sig;
    const void* gsig;
    void* dzinc;
    int64_t batch, L;
    int d;
    int64_t sig_stride;
    int scalar;
    hipStream_t stream;
    int nseg = 1;           // time segments per path; batch counts (path, segment) items
    int64_t lseg = 0;       // steps per segment (0: L)
    int from_points = 0;    // staged kernels of at most kPointFedMaxDim channels: inc is the plain path [paths][L + 1][d]
};

typedef hipError_t (*FwdFn)(const FwdParams&);
typedef hipError_t (*BwdFn)(const BwdParams&);

// D == 0: run-time dimension, packed layout; D == -1: run-time dimension, wide layout.  Exactly one of fwd / bwd is set.
struct KernelEntry {
    int is_f64, D, N, tail, k;
    int staged;      // 1: increments staged through LDS into VGPRs (wide layout, low occupancy)
    FwdFn fwd;
    BwdFn bwd;
    const char* name;
    int preferred;   // default partition of its shape
    int (*waves_per_simd)();   // register-limited residency of the kernel
    int stage_policy;          // which twin to launch: 0 general rules, 1 always the staged one, 2 never, 3 only when under-filled
    // staged forward instances: the same sweep for lead-lag increments (with a time channel iff D is odd), which
    // skips the letters a step cannot move; null when not compiled.  Needs an even FwdParams::lseg.
    FwdFn fwd_lead_lag = nullptr;
    // backward instances (staged, and scalar-fed ones with a subtree level below the lane's own letters): likewise; needs
    // an even number of steps per path and an even BwdParams::lseg.
    BwdFn bwd_lead_lag = nullptr;
};

// every generated instance file contributes one array
struct EntryList {
    const KernelEntry* entries;
    int count;
};

const EntryList* all_entry_lists(int* n_lists);   // defined in the generated registry

}  // namespace sigamd
