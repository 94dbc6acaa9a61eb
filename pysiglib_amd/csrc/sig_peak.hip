// Measured ceiling of the vector FMA pipes: independent multiply-adds, nothing else, at a chosen number of waves per
// SIMD.  The benchmark reports it beside the nominal peak: the sweeps of small batches run one wave per SIMD, and what
// a lone wave can issue is the ceiling that applies to them.  No counterpart in the reference.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <algorithm>

#include "../../include/cusig_amd.h"
#include "sig_host.h"

namespace sigamd {

// 16 accumulators (v[10:41] as 64-bit pairs, v10..v25 as 32-bit registers), 8 rounds: 128 independent FMAs per trip,
// all in the 8-byte encoding and on 8-byte boundaries
#define SIGAMD_ACC16(I) I(10) I(12) I(14) I(16) I(18) I(20) I(22) I(24) I(26) I(28) I(30) I(32) I(34) I(36) I(38) I(40)
#define SIGAMD_FMA64(n) "v_fma_f64 v[" #n ":" #n "+1], v[" #n ":" #n "+1], v[42:43], v[44:45]\n"
#define SIGAMD_FMA32(n) "v_fma_f32 v[" #n "], v[" #n "], v42, v44\n v_fma_f32 v[" #n "+1], v[" #n "+1], v42, v44\n"
#define SIGAMD_X8(X) X X X X X X X X
#define SIGAMD_CLOBBER "v10", "v11", "v12", "v13", "v14", "v15", "v16", "v17", "v18", "v19", "v20", "v21", "v22", "v23", "v24",     \
                       "v25", "v26", "v27", "v28", "v29", "v30", "v31", "v32", "v33", "v34", "v35", "v36", "v37", "v38", "v39",     \
                       "v40", "v41", "v42", "v43", "v44", "v45"

template <bool F64>
__global__ __launch_bounds__(256) void fma_peak_kernel(float* out, int trips)
{
    if (F64) asm volatile("v_mov_b32 v42, 0\n v_mov_b32 v43, 0x3ff00000\n v_mov_b32 v44, 0\n v_mov_b32 v45, 0\n" ::: SIGAMD_CLOBBER);
    else asm volatile("v_mov_b32 v42, 1.0\n v_mov_b32 v44, 0\n" ::: SIGAMD_CLOBBER);
    for (int t = 0; t < trips; ++t) {
        if (F64) asm volatile(".p2align 3\n" SIGAMD_X8(SIGAMD_ACC16(SIGAMD_FMA64)) ::: SIGAMD_CLOBBER);
        else asm volatile(".p2align 3\n" SIGAMD_X8(SIGAMD_ACC16(SIGAMD_FMA32)) ::: SIGAMD_CLOBBER);      // 256 FMAs per trip
    }
    if (trips < 0) out[threadIdx.x] = 1.0f;
}

template <bool F64>
static double measure(int waves_per_simd)
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    SIG_HIP(hipGetDeviceProperties(&prop, dev));
    const int blocks = prop.multiProcessorCount * waves_per_simd;       // a block of 256 threads: one wave on each SIMD of a CU
    const int trips = 20000;     // ~5 ms a launch: long enough for the clocks to settle under the load
    float* out = nullptr;
    SIG_HIP(hipMalloc(&out, 1024 * sizeof(float)));
    hipEvent_t e0 = nullptr, e1 = nullptr;
    double best = 0;
    try {
        SIG_HIP(hipEventCreate(&e0));
        SIG_HIP(hipEventCreate(&e1));
        for (int rep = 0; rep < 4; ++rep) {       // the first launch warms the clocks
            SIG_HIP(hipEventRecord(e0, nullptr));
            hipLaunchKernelGGL((fma_peak_kernel<F64>), dim3(blocks), dim3(256), 0, nullptr, out, trips);
            SIG_HIP(hipEventRecord(e1, nullptr));
            SIG_HIP(hipEventSynchronize(e1));
            float ms = 0;
            SIG_HIP(hipEventElapsedTime(&ms, e0, e1));
            const double fmas = double(blocks) * 256 * trips * (F64 ? 128 : 256);
            if (rep) best = std::max(best, 2 * fmas / (ms * 1e-3) / 1e12);
        }
    } catch (...) {
        if (e0) (void)hipEventDestroy(e0);
        if (e1) (void)hipEventDestroy(e1);
        (void)hipFree(out);
        throw;
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    (void)hipFree(out);
    return best;
}

}  // namespace sigamd

extern "C" CUSIG_AMD_API int cusig_amd_measure_fma_peak(int is_f64, int waves_per_simd, double* tflops) noexcept
{
    using namespace sigamd;
    return guarded([&] {
        if (!tflops || waves_per_simd < 1 || waves_per_simd > 8) throw std::invalid_argument("cusig_amd_measure_fma_peak: 1 to 8 waves per SIMD");
        SIG_HIP(hipDeviceSynchronize());
        *tflops = is_f64 ? measure<true>(waves_per_simd) : measure<false>(waves_per_simd);
    });
}
