// Adjoint of the Chen product: kernels and their launcher, shared by sig_combine_backprop, sig_join_backprop, the
// tensor logarithm's backward pass and the time-split signature backward.
#include "sig_chen_adjoint.h"

#include <atomic>
#include <type_traits>

#include "sig_kernels.h"
#include "sig_chen_stream.h"

namespace sigamd {

// four consecutive elements with the alignment of one
template <typename T>
struct alignas(sizeof(T)) Quad {
    T v[4];
};
constexpr int kCombChunk = 256;
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
    int identity, int64_t dc_share, int64_t dc_stride, int dc_off, int families, int only_b)
{
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        for (I r = I(xcd_block_2d().x) * kBlock + threadIdx.x; r < init_len; r += I(gridDim.x) * kBlock) {
            const T v = identity ? dC[(b / dc_share) * dc_stride + dc_off + r] : T(0);
            if (!only_b) dA[b * stride + off + r] = (identity & 1) ? v : T(0);
            if (families > 1 || only_b) dB[b * stride + off + r] = (identity & 2) ? v : T(0);
        }
    }
}

template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void sig_combine_bwd_kernel(
    const T* __restrict__ dC, T* __restrict__ dA, T* __restrict__ dB, const T* __restrict__ A,
    const T* __restrict__ B, int64_t batch, CombBwdPlan<I> plan, int64_t stride, int off, int identity,
    int64_t dc_share, int64_t dc_stride, int dc_off, int families, int only_b)
{
    const int N = plan.degree;
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        const T* g = dC + (b / dc_share) * dc_stride + dc_off;
        for (I it = I(xcd_block_2d().x) * kBlock + threadIdx.x; it < I(families) * plan.items; it += I(gridDim.x) * kBlock) {
            const bool fam_b = only_b || it >= plan.items;
            const I i2 = it >= plan.items ? it - plan.items : it;
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
            if (plan.parts[t] == 1) *dst = ((identity >> int(fam_b)) & 1 ? g[r] : T(0)) + sum;
            else dev_add(dst, sum);
            if (off && it == 0) {
                if (!only_b) dA[b * stride] = T(0);
                if (families > 1 || only_b) dB[b * stride] = T(0);
            }
        }
    }
}

// test hook (defined in sig_api.hip): 0 = streaming kernels for rows of at least kStreamMinCoef coefficients,
// 1 = streaming kernels wherever they apply, 2 = item-per-word kernels only
extern std::atomic<int> g_chen_adjoint_mode;
constexpr uint64_t kStreamMinCoef = 4096;
constexpr uint64_t kStreamLdsEntries = 6144;      // 48 KB of float64

// the item-per-word kernels on the signature truncated at `degree` (rows keep their stride): both factors, or one
template <typename T>
static void launch_combine_bwd_items(const T* dC, T* dA, T* dB, const T* A, const T* B, uint64_t batch, uint64_t dimension,
                                     uint64_t degree, const SigShape& s, hipStream_t stream, int identity,
                                     const SharedRows& dc, int families, int only_b)
{
    launch_indexed(3 * s.n_coef + 1024, 1, batch, [&](auto ix, dim3) {      // 2 * items <= 2 n (1 + degree / kCombChunk)
        using I = decltype(ix);
        const CombBwdPlan<I> plan = make_comb_plan<I>(dimension, degree);
        if (plan.init_len > 0)
            launch_indexed(0, uint64_t(plan.init_len), batch, [&](auto, dim3 grid) {
                hipLaunchKernelGGL((sig_combine_bwd_init_kernel<T, I>), grid, dim3(kBlock), 0, stream, dC, dA, dB,
                                   int64_t(batch), plan.init_len, int64_t(s.stride), s.off, identity, dc.share, dc.stride,
                                   dc.off, families, only_b);
            });
        launch_indexed(0, uint64_t(families) * uint64_t(plan.items), batch, [&](auto, dim3 grid) {
            hipLaunchKernelGGL((sig_combine_bwd_kernel<T, I>), grid, dim3(kBlock), 0, stream, dC, dA, dB, A, B, int64_t(batch),
                               plan, int64_t(s.stride), s.off, identity, dc.share, dc.stride, dc.off, families, only_b);
        });
    });
}

// LDS of the right factor's kernel when it folds exp(z): one slot per lane and letter
template <typename T>
static bool right_fold_fits(uint64_t dimension)
{
    return dimension * uint64_t(kBlock) * sizeof(T) <= uint64_t(64) << 10;
}

template <typename T, int QL = 0, int REL = 1>
static void launch_right_stream(const RightPlan& rp, const T* dC, T* dB, const T* A, uint64_t batch, const SigShape& s,
                                hipStream_t stream, int identity, const SharedRows& dc, const ExpFold<T>* fold)
{
    if constexpr (QL <= kRightMaxLow && REL <= kRightMaxRel) {
        if (rp.qe - 1 != QL) return launch_right_stream<T, QL + 1, REL>(rp, dC, dB, A, batch, s, stream, identity, dc, fold);
        if (rp.rel != REL) return launch_right_stream<T, QL, REL + 1>(rp, dC, dB, A, batch, s, stream, identity, dc, fold);
        const uint64_t waves = (uint64_t(rp.words) + kWave - 1) / kWave;
        const dim3 grid{unsigned((waves + kWavesPerBlock - 1) / kWavesPerBlock), unsigned(std::min<uint64_t>(batch, 65535)), 1};
        FoldScale<T> fs{};
        if (fold) {
            double fact = 1.0;
            for (int t = 1; t <= rp.qe; ++t) fact *= double(t);
            for (int D = 0; D <= REL; ++D) {
                if (D) fact *= double(rp.qe + D);
                fs.inv_level[D] = T(1.0 / double(rp.qe + D));
                fs.inv_fact[D] = T(1.0 / fact);
            }
            hipLaunchKernelGGL((chen_adjoint_right_kernel<T, QL, REL, true>), grid, dim3(kBlock),
                               size_t(rp.d) * kBlock * sizeof(T), stream, dC, dB, A, int64_t(batch), rp, int64_t(s.stride), s.off,
                               identity, dc.share, dc.stride, dc.off, fold->z, fold->dz, fs);
        } else {
            hipLaunchKernelGGL((chen_adjoint_right_kernel<T, QL, REL, false>), grid, dim3(kBlock), 0, stream, dC, dB, A,
                               int64_t(batch), rp, int64_t(s.stride), s.off, identity, dc.share, dc.stride, dc.off,
                               (const T*)nullptr, (T*)nullptr, fs);
        }
    }
}

// launches the adjoint of the Chen product on `stream`
template <typename T>
void launch_combine_bwd(const T* dC, T* dA, T* dB, const T* A, const T* B, uint64_t batch, uint64_t dimension,
                        uint64_t degree, const SigShape& s, hipStream_t stream, int identity, SharedRows dc, int families,
                        ExpFold<T>* fold)
{
    if (dc.stride < 0) { dc.stride = int64_t(s.stride); dc.off = s.off; }
    if (fold) fold->level = int(degree);
    const int ida = identity & 1, idb = (identity >> 1) & 1;
    if (degree > uint64_t(kCombMaxLevels)) throw std::runtime_error("sig_combine_backprop_cuda: degree too high");
    const int mode = g_chen_adjoint_mode;
    const bool streaming = mode != 2 && (mode == 1 || s.n_coef >= kStreamMinCoef) && dimension >= 2 && degree >= 2 &&
                           degree <= uint64_t(kStreamMaxLevels) && s.n_coef < (uint64_t(1) << 28) &&
                           !g_force_wide_index;
    LeftPlan lp;
    RowsPlan wp;
    RightPlan rp;
    const bool rows = streaming && make_rows_plan(wp, dimension, degree, kStreamLdsEntries);
    const bool left = rows || (streaming && make_left_plan(lp, dimension, degree, kStreamLdsEntries));
    const bool right = streaming && families > 1 && make_right_plan(rp, dimension, degree);
    if (!left && !right) {
        launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, degree, s, stream, identity, dc, families, 0);
        return;
    }
    // left factor: words shorter than the blocks' own take their low-level terms from the truncated problem first
    if (!left) {
        launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, degree, s, stream, identity, dc, 1, 0);
    } else if (rows) {
        if (wp.np >= 2)
            launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, uint64_t(wp.np), s, stream, identity, dc, 1, 0);
        const uint64_t groups = (uint64_t(wp.units) + uint64_t(wp.upb) - 1) / uint64_t(wp.upb);
        const dim3 grid{unsigned(groups), unsigned(std::min<uint64_t>(batch, 65535)), 1};
        const size_t lds = (size_t(wp.bs) + 2 * size_t(wp.targets) + size_t(wp.img)) * sizeof(T);
        const int kt = int((wp.top + kBlock - 1) / kBlock), ks = int((wp.targets + kBlock - 1) / kBlock);
        auto go3 = [&](auto dc_, auto kt_, auto ks_) {
            hipLaunchKernelGGL((chen_adjoint_left_rows_kernel<T, decltype(dc_)::value, decltype(kt_)::value, decltype(ks_)::value>),
                               grid, dim3(kBlock), lds, stream, dC, dA, B, int64_t(batch), wp, int64_t(s.stride), s.off, ida,
                               dc.share, dc.stride, dc.off);
        };
        auto go2 = [&](auto dc_, auto ks_) {
            if (kt <= 2) go3(dc_, std::integral_constant<int, 2>(), ks_);
            else if (kt <= 4) go3(dc_, std::integral_constant<int, 4>(), ks_);
            else go3(dc_, std::integral_constant<int, kRowsMaxTop>(), ks_);
        };
        // owned entries per thread: more than one only for few channels (targets ~ top / (d - 1))
        auto go = [&](auto dc_) {
            constexpr int DC = decltype(dc_)::value;
            if (ks <= 1) go2(dc_, std::integral_constant<int, 1>());
            else if constexpr (DC <= 8) {
                if (ks <= 2) go2(dc_, std::integral_constant<int, 2>());
                else if constexpr (DC <= 4) go2(dc_, std::integral_constant<int, kRowsMaxLow>());
                else throw std::logic_error("sig_combine_backprop_cuda: kernel plan");
            } else throw std::logic_error("sig_combine_backprop_cuda: kernel plan");
        };
        const uint64_t d = dimension;
        if (d <= 4) go(std::integral_constant<int, 4>());
        else if (d <= 8) go(std::integral_constant<int, 8>());
        else if (d <= 12) go(std::integral_constant<int, 12>());
        else if (d <= 16) go(std::integral_constant<int, 16>());
        else go(std::integral_constant<int, 32>());
    } else {
        if (lp.np >= 2)
            launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, uint64_t(lp.np), s, stream, identity, dc, 1, 0);
        const uint64_t groups = (uint64_t(lp.units) + uint64_t(lp.upb) - 1) / uint64_t(lp.upb);
        const dim3 grid{unsigned(groups), unsigned(std::min<uint64_t>(batch, 65535)), 1};
        const size_t lds = (size_t(lp.xs) + size_t(lp.bs)) * sizeof(T);
        auto go = [&](auto kx) {
            hipLaunchKernelGGL((chen_adjoint_left_kernel<T, decltype(kx)::value>), grid, dim3(kBlock), lds, stream, dC, dA, B,
                               int64_t(batch), lp, int64_t(s.stride), s.off, ida, dc.share, dc.stride, dc.off);
        };
        const uint32_t per = (lp.xs + kBlock - 1) / kBlock;      // entries of a unit per thread
        if (per <= 4) go(std::integral_constant<int, 4>());
        else if (per <= 8) go(std::integral_constant<int, 8>());
        else if (per <= 12) go(std::integral_constant<int, 12>());
        else if (per <= 16) go(std::integral_constant<int, 16>());
        else go(std::integral_constant<int, 24>());
    }
    if (families < 2) return;
    if (!right) {
        launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, degree, s, stream, identity, dc, 1, 1);
    } else {
        if (rp.qe >= 2)
            launch_combine_bwd_items<T>(dC, dA, dB, A, B, batch, dimension, uint64_t(rp.qe - 1), s, stream, identity, dc, 1, 1);
        const bool folding = fold && idb == 1 && rp.rel >= 1 && right_fold_fits<T>(dimension);
        if (folding) fold->level = rp.qe;
        launch_right_stream<T>(rp, dC, dB, A, batch, s, stream, idb, dc, folding ? fold : nullptr);
    }
}

template void launch_combine_bwd<float>(const float*, float*, float*, const float*, const float*, uint64_t, uint64_t,
                                        uint64_t, const SigShape&, hipStream_t, int, SharedRows, int, ExpFold<float>*);
template void launch_combine_bwd<double>(const double*, double*, double*, const double*, const double*, uint64_t,
                                         uint64_t, uint64_t, const SigShape&, hipStream_t, int, SharedRows, int,
                                         ExpFold<double>*);

}  // namespace sigamd
