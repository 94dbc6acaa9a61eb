// Signature sweeps of run-time degree (17 .. 64) for 2, 3 or 4 augmented channels; defined in sig_deep.hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "sig_registry.h"

namespace sigamd {

constexpr int kDeepMaxDegree = 64;      // as the reference's run-time-degree kernels (siglib/cusig/cu_signature.cu:400)

// whether launch_deep_fwd / launch_deep_bwd serve (augmented dimension, degree)
bool deep_supported(uint64_t d, uint64_t degree);

// whether a launch for `batch` paths fits the grid limits (to be checked before anything is enqueued)
bool deep_fits(uint64_t d, uint64_t degree, uint64_t batch);

// whole-path sweeps (nseg must be 1); p.d is the augmented dimension
template <typename T>
hipError_t launch_deep_fwd(const FwdParams& p, int degree);
template <typename T>
hipError_t launch_deep_bwd(const BwdParams& p, int degree);

}  // namespace sigamd
