// Adjoint of the Chen product, shared by sig_combine_backprop, sig_join_backprop and the tensor logarithm's backward
// pass, plus the row layout helper of the signature-shaped operators.
#pragma once
#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>

#include "sig_host.h"
#include "sig_kernels.h"

namespace sigamd {

// Adjoint of C = A (x) B (siglib/cpsig/cp_sig_combine.h:126-176), scalar-free rows:
//   dA_t[w] = dC_t[w] + sum_{m=1..N-t} sum_{v in d^m} dC_{t+m}[w v] * B_m[v]        (contiguous block of dC)
//   dB_t[w] = dC_t[w] + sum_{k=1..N-t} sum_{u in d^k} dC_{t+k}[u w] * A_k[u]        (stride d^t in dC)
// Both sums run over the first S_t = d + .. + d^(N-t) entries x of the other factor's row (its levels 1..N-t laid
// end to end).  Outputs of low levels have long sums, so a sum is cut into parts of kCombChunk entries; a work
// item is (family, level t, part, word w), words fastest.  Levels with one part are stored directly, the others
// are set to dC by sig_combine_bwd_init_kernel first and receive their parts through atomics.
// identity = 0 drops the dC_t[w] terms: the adjoint of the product without its "+ A + B" part, sum_l A_l (x) B_{t-l},
// which is what the tensor logarithm is built from.
// The rows of dC may be laid out differently from the others (stride dc_stride, dc_off leading slots) and shared:
// item b reads row b / dc_share.  families = 1 computes dA only (dB and A are not touched).
// four consecutive elements with the alignment of one
template <typename T>
struct alignas(sizeof(T)) Quad {
    T v[4];
};
constexpr int kCombChunk = 256;
constexpr int kCombMaxLevels = 64;
template <typename I>
struct CombBwdPlan {
    int degree;
    I items;                            // work items of one family
    I lo[kCombMaxLevels + 2];           // lo[t]: start of level t in a scalar-free row, t = 1 .. degree + 1
    I item_start[kCombMaxLevels + 2];   // first work item of level t
    I parts[kCombMaxLevels + 2];        // parts per word of level t (>= 1)
    I init_len;                         // coefficients (a prefix of the row) whose levels have several parts
};

template <typename I>
static CombBwdPlan<I> make_comb_plan(uint64_t d, uint64_t degree)
{
    CombBwdPlan<I> p{};
    p.degree = int(degree);
    uint64_t lo = 0, sz = d;
    for (uint64_t t = 1; t <= degree + 1; ++t) {
        p.lo[t] = I(lo);
        lo += sz;
        if (t <= degree) sz *= d;
    }
    uint64_t items = 0;
    p.init_len = 0;
    for (uint64_t t = 1; t <= degree; ++t) {
        const uint64_t s_t = uint64_t(p.lo[degree - t + 1]);          // d + .. + d^(degree - t)
        const uint64_t parts = s_t == 0 ? 1 : (s_t + kCombChunk - 1) / kCombChunk;
        p.item_start[t] = I(items);
        p.parts[t] = I(parts);
        items += parts * (uint64_t(p.lo[t + 1]) - uint64_t(p.lo[t]));
        if (parts > 1) p.init_len = p.lo[t + 1];
    }
    p.item_start[degree + 1] = I(items);
    p.items = I(items);
    return p;
}

template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void sig_combine_bwd_init_kernel(
    const T* __restrict__ dC, T* __restrict__ dA, T* __restrict__ dB, int64_t batch, I init_len, int64_t stride, int off,
    int identity, int64_t dc_share, int64_t dc_stride, int dc_off, int families)
{
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        for (I r = I(xcd_block_2d().x) * kBlock + threadIdx.x; r < init_len; r += I(gridDim.x) * kBlock) {
            const T v = identity ? dC[(b / dc_share) * dc_stride + dc_off + r] : T(0);
            dA[b * stride + off + r] = v;
            if (families > 1) dB[b * stride + off + r] = v;
        }
    }
}

template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void sig_combine_bwd_kernel(
    const T* __restrict__ dC, T* __restrict__ dA, T* __restrict__ dB, const T* __restrict__ A,
    const T* __restrict__ B, int64_t batch, CombBwdPlan<I> plan, int64_t stride, int off, int identity,
    int64_t dc_share, int64_t dc_stride, int dc_off, int families)
{
    const int N = plan.degree;
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        const T* g = dC + (b / dc_share) * dc_stride + dc_off;
        for (I it = I(xcd_block_2d().x) * kBlock + threadIdx.x; it < I(families) * plan.items; it += I(gridDim.x) * kBlock) {
            const bool fam_b = it >= plan.items;
            const I i2 = fam_b ? it - plan.items : it;
            int t = 1;
            while (t < N && i2 >= plan.item_start[t + 1]) ++t;
            const I sz_t = plan.lo[t + 1] - plan.lo[t];
            const I local = i2 - plan.item_start[t];
            const I q = local / sz_t;
            const I w = local - q * sz_t;
            const I s_t = plan.lo[N - t + 1];
            const I x0 = q * kCombChunk;
            const I x1 = x0 + kCombChunk < s_t ? x0 + kCombChunk : s_t;
            const T* other = (fam_b ? A : B) + b * stride + off;      // the factor the sum runs over
            T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
            for (int m = 1; m <= N - t; ++m) {
                const I seg0 = plan.lo[m] > x0 ? plan.lo[m] : x0;
                const I seg1 = plan.lo[m + 1] < x1 ? plan.lo[m + 1] : x1;
                if (seg0 >= seg1) continue;
                const T* up = g + plan.lo[t + m];                     // level t + m of dC
                if (!fam_b) {
                    const T* blockp = up + w * (plan.lo[m + 1] - plan.lo[m]) - plan.lo[m];    // words w v
                    I x = seg0;
                    for (; x + 4 <= seg1; x += 4) {      // all loads are issued before the first product needs one
                        // a lane walks a block of its own, so every load costs it a cache access of its own: take the
                        // four consecutive entries in wide loads (element alignment is all that is known)
                        const Quad<T> gq = *reinterpret_cast<const Quad<T>*>(blockp + x);
                        const Quad<T> oq = *reinterpret_cast<const Quad<T>*>(other + x);
                        s0 = fmadd(gq.v[0], oq.v[0], s0);
                        s1 = fmadd(gq.v[1], oq.v[1], s1);
                        s2 = fmadd(gq.v[2], oq.v[2], s2);
                        s3 = fmadd(gq.v[3], oq.v[3], s3);
                    }
                    for (; x < seg1; ++x) s0 = fmadd(blockp[x], other[x], s0);
                } else {
                    const T* strided = up + w;                         // words u w: index u * d^t + w
                    I x = seg0;
                    for (; x + 4 <= seg1; x += 4) {
                        const T* sp = strided + (x - plan.lo[m]) * sz_t;
                        const T g0 = sp[0], g1 = sp[sz_t], g2 = sp[2 * sz_t], g3 = sp[3 * sz_t];
                        const Quad<T> oq = *reinterpret_cast<const Quad<T>*>(other + x);      // the same four for the whole wave
                        s0 = fmadd(g0, oq.v[0], s0);
                        s1 = fmadd(g1, oq.v[1], s1);
                        s2 = fmadd(g2, oq.v[2], s2);
                        s3 = fmadd(g3, oq.v[3], s3);
                    }
                    for (; x < seg1; ++x) s0 = fmadd(strided[(x - plan.lo[m]) * sz_t], other[x], s0);
                }
            }
            const I r = plan.lo[t] + w;
            T* dst = (fam_b ? dB : dA) + b * stride + off + r;
            const T sum = (s0 + s1) + (s2 + s3);
            if (plan.parts[t] == 1) *dst = (identity ? g[r] : T(0)) + sum;
            else dev_add(dst, sum);
            if (off && it == 0) {
                dA[b * stride] = T(0);
                if (families > 1) dB[b * stride] = T(0);
            }
        }
    }
}

struct SigShape {
    uint64_t n_coef, stride;
    int off;
};

static SigShape sig_shape(uint64_t dimension, uint64_t degree, bool scalar_term, const char* who)
{
    if (dimension == 0) throw std::invalid_argument(std::string(who) + " received dimension 0");
    if (dimension > 0x3fffffff || degree > 0x7fffffff) throw std::invalid_argument(std::string(who) + ": shape out of range");
    const uint64_t full = sig_length_u64(dimension, degree);
    if (full == 0) throw std::overflow_error("signature length overflows 64 bits");
    SigShape s;
    s.n_coef = full - 1;
    s.stride = scalar_term ? full : full - 1;
    s.off = scalar_term ? 1 : 0;
    return s;
}

// how the rows of dC are found when they differ from the other operands' layout
struct SharedRows {
    int64_t share = 1;      // consecutive items reading one row
    int64_t stride = -1;    // < 0: same stride and offset as the other operands
    int off = 0;
};

// launches the adjoint of the Chen product (both kernels) on `stream`
template <typename T>
static void launch_combine_bwd(const T* dC, T* dA, T* dB, const T* A, const T* B, uint64_t batch, uint64_t dimension,
                               uint64_t degree, const SigShape& s, hipStream_t stream, int identity = 1,
                               SharedRows dc = SharedRows(), int families = 2)
{
    if (dc.stride < 0) { dc.stride = int64_t(s.stride); dc.off = s.off; }
    if (degree > uint64_t(kCombMaxLevels)) throw std::runtime_error("sig_combine_backprop_cuda: degree too high");
    launch_indexed(3 * s.n_coef + 1024, 1, batch, [&](auto ix, dim3) {      // 2 * items <= 2 n (1 + degree / kCombChunk)
        using I = decltype(ix);
        const CombBwdPlan<I> plan = make_comb_plan<I>(dimension, degree);
        if (plan.init_len > 0)
            launch_indexed(0, uint64_t(plan.init_len), batch, [&](auto, dim3 grid) {
                hipLaunchKernelGGL((sig_combine_bwd_init_kernel<T, I>), grid, dim3(kBlock), 0, stream, dC, dA, dB,
                                   int64_t(batch), plan.init_len, int64_t(s.stride), s.off, identity, dc.share, dc.stride,
                                   dc.off, families);
            });
        launch_indexed(0, uint64_t(families) * uint64_t(plan.items), batch, [&](auto, dim3 grid) {
            hipLaunchKernelGGL((sig_combine_bwd_kernel<T, I>), grid, dim3(kBlock), 0, stream, dC, dA, dB, A, B, int64_t(batch),
                               plan, int64_t(s.stride), s.off, identity, dc.share, dc.stride, dc.off, families);
        });
    });
}

}  // namespace sigamd
