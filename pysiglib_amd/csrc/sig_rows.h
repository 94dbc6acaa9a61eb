// Sweeps for many channels (more than 32) at degrees 3 .. 8; defined in sig_rows.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sig_registry.h"

namespace sigamd {

// whether launch_rows_bwd serves (element size, augmented dimension, degree)
bool rows_bwd_supported(size_t elem_bytes, uint64_t d, uint64_t degree);

// whether a launch for `batch` paths fits the grid limits (to be checked before anything is enqueued)
bool rows_bwd_fits(size_t elem_bytes, uint64_t d, uint64_t degree, uint64_t batch);

// whole-path sweeps (p.nseg must be 1, p.inc holds increments); p.d is the augmented dimension
template <typename T>
hipError_t launch_rows_bwd(const BwdParams& p, int degree);
template <typename T>
hipError_t launch_rows_fwd(const FwdParams& p, int degree);

}  // namespace sigamd
