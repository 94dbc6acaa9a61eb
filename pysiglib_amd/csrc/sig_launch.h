// Launch wrappers instantiated once per (T, D, N, TAIL, K).
#pragma once
#include "sig_kernels.h"
#include "sig_registry.h"

namespace sigamd {

constexpr int64_t kMaxGridX = 2147483647LL;
constexpr size_t kMaxDynLds = 64 * 1024;
constexpr size_t kMaxLdsPerBlock = 160 * 1024;

// dynamic LDS above 64 KB has to be requested once per kernel
template <typename Kern>
hipError_t allow_lds(Kern kern, size_t bytes)
{
    if (bytes <= kMaxDynLds) return hipSuccess;
    if (bytes > kMaxLdsPerBlock) return hipErrorInvalidConfiguration;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, int(bytes));
}

template <typename T, int D, int N, int TAIL, int K, bool ZL, int LL = 0>
hipError_t launch_tree_fwd(const FwdParams& p)
{
    if (LL != 0 && ((p.lseg & 1) || p.from_points)) return hipErrorInvalidConfiguration;    // ranges must start on even steps
    const TreeGeom g = make_geom(p.d, N - TAIL, K, D != 0);
    if (D < 0 && !g.wide) return hipErrorInvalidConfiguration;     // the kernel was compiled for the wide layout
    const int64_t waves = total_waves(g, p.batch);
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks < 1 || blocks > kMaxGridX) return hipErrorInvalidConfiguration;
    static_assert(!ZL || D <= 0 || IncRing<T, (D > 0 ? D : 1), 1>::kPoints == (D <= kPointFedMaxDim),
                  "the ring's point-fed mode and the host's limit must agree");
    if (p.from_points && !(ZL && D > 0 && D <= kPointFedMaxDim)) return hipErrorInvalidConfiguration;
    size_t lds = 0;
    if (ZL) {
        if (!g.wide) return hipErrorInvalidConfiguration;
        lds = size_t(kWavesPerBlock) * IncRing<T, (D > 0 ? D : 1), 1>::ELEMS * sizeof(T);
        hipError_t e = allow_lds(tree_fwd_kernel<T, D, N, TAIL, K, ZL, LL>, lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((tree_fwd_kernel<T, D, N, TAIL, K, ZL, LL>), dim3((unsigned)blocks), dim3(kBlock), lds, p.stream,
                       static_cast<const T*>(p.inc), static_cast<T*>(p.out), p.batch, p.L, p.d,
                       p.out_stride, p.scalar, p.nseg, p.lseg, p.nonfinite, (ZL && D > 0 && D <= kPointFedMaxDim) ? p.from_points : 0);
    return hipGetLastError();
}

// resident waves per SIMD of the forward kernel (register-limited)
template <typename T, int D, int N, int TAIL, int K, bool ZL>
int fwd_waves_per_simd()
{
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, tree_fwd_kernel<T, D, N, TAIL, K, ZL>, kBlock, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 1;
    }
    return blocks < 1 ? 1 : blocks;
}

// resident waves per SIMD of the backward kernel (register-limited; its LDS tiles never limit below that)
template <typename T, int D, int N, int TAIL, int K, bool ZL>
int bwd_waves_per_simd()
{
    int blocks = 0;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&blocks, tree_bwd_kernel<T, D, N, TAIL, K, ZL>, kBlock, 0) != hipSuccess) {
        (void)hipGetLastError();
        return 1;
    }
    return blocks < 1 ? 1 : blocks;
}

template <typename T, int D, int N, int TAIL, int K, bool ZL, int LL = 0>
hipError_t launch_tree_bwd(const BwdParams& p)
{
    static_assert(LL == 0 || (D >= 4 && (ZL || TAIL >= 2)), "the lead-lag sweep needs a compile-time dimension");
    // the lead-lag sweep reads a step's parity off its position in the range: ranges must be even and start even
    if (LL != 0 && ((p.L & 1) || (p.nseg > 1 && (p.lseg & 1)) || p.from_points)) return hipErrorInvalidConfiguration;
    if (p.from_points && !(ZL && D > 0 && D <= kPointFedMaxDim)) return hipErrorInvalidConfiguration;
    const TreeGeom g = make_geom(p.d, N - TAIL, K, D != 0);
    if (D < 0 && !g.wide) return hipErrorInvalidConfiguration;     // the kernel was compiled for the wide layout
    const int64_t waves = total_waves(g, p.batch);
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks < 1 || blocks > kMaxGridX) return hipErrorInvalidConfiguration;
    size_t lds;
    int use_lds = 1;
    using Plan = RedPlan<T, D, TAIL, K, ZL>;
    if (Plan::steps(p.d) > 0) {
        lds = size_t(kWavesPerBlock) * size_t(Plan::tile_elems(p.d)) * sizeof(T);
    } else if (g.ppw == 1) {
        // wider than any tile: the letters of a step pass through a tile of kRows rows in groups
        use_lds = 2;
        lds = size_t(kWavesPerBlock) * size_t(Plan::kRows) * kRedStride * sizeof(T);
    } else {
        lds = size_t(kWavesPerBlock) * size_t(g.ppw) * size_t(p.d) * sizeof(T);
        if (lds > kMaxDynLds) { use_lds = 0; lds = 0; }
    }
    if (ZL) {
        if (!g.wide) return hipErrorInvalidConfiguration;
        lds += size_t(kWavesPerBlock) * IncRing<T, (D > 0 ? D : 1), -1>::ELEMS * sizeof(T);
    }
    {
        hipError_t e = allow_lds(tree_bwd_kernel<T, D, N, TAIL, K, ZL, LL>, lds);
        if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL((tree_bwd_kernel<T, D, N, TAIL, K, ZL, LL>), dim3((unsigned)blocks), dim3(kBlock), lds, p.stream,
                       static_cast<const T*>(p.inc), static_cast<const T*>(p.sig),
                       static_cast<const T*>(p.gsig), static_cast<T*>(p.dzinc), p.batch, p.L, p.d,
                       p.sig_stride, p.scalar, use_lds, p.nseg, p.lseg > 0 ? p.lseg : p.L,
                       (ZL && D > 0 && D <= kPointFedMaxDim) ? p.from_points : 0);
    return hipGetLastError();
}

}  // namespace sigamd
