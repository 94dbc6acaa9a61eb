// Operators either side of the signature sweep, behind the reference's entry points:
//   sig_combine_cuda_{f,d}, sig_combine_backprop_cuda_{f,d}   (siglib/cusig/cu_sig_combine.cu:157-337)
//   transform_path_cuda_{f,d}, transform_path_backprop_cuda_{f,d} (siglib/cusig/cu_path_transforms.cu:48-205)
//   linear_sig_cuda_{f,d}, sig_join_cuda_{f,d}, sig_join_backprop_cuda_{f,d} (siglib/cusig/cusig.h:929-987; arithmetic of
//   siglib/cpsig/cp_sig_join.h:36-238 and linear_sig_deriv_to_increment_deriv, siglib/cpsig/cp_sig_combine.h:232-263)
// The Chen product itself is the kernel the time-segmented forward sweep folds its pieces with.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>

#include "../../include/cusig_amd.h"
#include "sig_host.h"
#include "sig_kernels.h"
#include "sig_chen_adjoint.h"

namespace sigamd {

// Materialised lead-lag / time augmentation: point i of the lead-lag path has lag = x[i/2] and
// lead = x[i/2 + (i odd)]; time is the last channel, i * end_time / (len_eff - 1)
// (siglib/cpsig/cp_path_transforms.h:36-142).  One thread per output element of a path; `dtd` divides by the
// transformed dimension.
constexpr int kTransformBatch = 4;      // elements per thread whose loads are in flight together
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void transform_path_kernel(
    const T* __restrict__ in, T* __restrict__ out, int64_t batch, I len, I d, DivBy<I> dtd, int time_aug, int lead_lag, T scale)
{
    const I td = I(dtd.d);
    const I tl = lead_lag ? 2 * len - 1 : len;
    const I per = tl * td;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = in + b * int64_t(len) * int64_t(d);
        T* o = out + b * int64_t(per);
        // kTransformBatch elements per thread, a grid apart, all loads before the first store
        const I step = I(gridDim.x) * kBlock;
        for (I e0 = I(blockIdx.x) * kBlock + threadIdx.x; e0 < per; e0 += kTransformBatch * step) {
            T v[kTransformBatch];
#pragma unroll
            for (int k = 0; k < kTransformBatch; ++k) {
                const I e = e0 + I(k) * step;
                const I ec = e < per ? e : per - 1;
                const I i = dtd.quot(ec);
                const I c = ec - i * td;
                // branch-free: the time channel loads element 0 and discards it
                const bool is_time = time_aug && c == td - 1;
                const I lag = (i >> 1) * d + c, lead = ((i >> 1) + (i & 1)) * d + (c - d);
                const I src = is_time ? I(0) : (!lead_lag ? i * d + c : (c < d ? lag : lead));
                const T raw = x[src];
                v[k] = is_time ? T(i) * scale : raw;
            }
#pragma unroll
            for (int k = 0; k < kTransformBatch; ++k) {
                const I e = e0 + I(k) * step;
                if (e < per) o[e] = v[k];
            }
        }
    }
}

// Adjoint of the augmentation: a raw point collects the gradient of every transformed point that copies it;
// the time channel has no raw counterpart (siglib/cpsig/cp_path_transforms.h:182-243).  `dd` divides by the raw
// dimension.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void transform_path_bwd_kernel(
    const T* __restrict__ derivs, T* __restrict__ out, int64_t batch, I len, DivBy<I> dd, int time_aug, int lead_lag)
{
    const I d = I(dd.d);
    const I td = (lead_lag ? 2 * d : d) + (time_aug ? 1 : 0);
    const I tl = lead_lag ? 2 * len - 1 : len;
    const I per = len * d;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* g = derivs + b * int64_t(tl) * int64_t(td);
        T* o = out + b * int64_t(per);
        for (I e = I(blockIdx.x) * kBlock + threadIdx.x; e < per; e += I(gridDim.x) * kBlock) {
            const I k = dd.quot(e);
            const I j = e - k * d;
            T v;
            if (!lead_lag) {
                v = g[k * td + j];
            } else {
                v = g[(2 * k) * td + j] + g[(2 * k) * td + d + j];
                if (k + 1 < len) v += g[(2 * k + 1) * td + j];
                if (k >= 1) v += g[(2 * k - 1) * td + d + j];
            }
            o[e] = v;
        }
    }
}

// 1/k for k = 0 .. 64 (entry 0 unused): the kernels below divide by small integers once per letter, and an FP64
// division costs some thirty instructions
constexpr int kExpMaxDegree = 64;
__constant__ double kRcp[kExpMaxDegree + 1] = {
    0.0, 1.0 / 1, 1.0 / 2, 1.0 / 3, 1.0 / 4, 1.0 / 5, 1.0 / 6, 1.0 / 7, 1.0 / 8, 1.0 / 9, 1.0 / 10, 1.0 / 11,
    1.0 / 12, 1.0 / 13, 1.0 / 14, 1.0 / 15, 1.0 / 16, 1.0 / 17, 1.0 / 18, 1.0 / 19, 1.0 / 20, 1.0 / 21, 1.0 / 22,
    1.0 / 23, 1.0 / 24, 1.0 / 25, 1.0 / 26, 1.0 / 27, 1.0 / 28, 1.0 / 29, 1.0 / 30, 1.0 / 31, 1.0 / 32, 1.0 / 33,
    1.0 / 34, 1.0 / 35, 1.0 / 36, 1.0 / 37, 1.0 / 38, 1.0 / 39, 1.0 / 40, 1.0 / 41, 1.0 / 42, 1.0 / 43, 1.0 / 44,
    1.0 / 45, 1.0 / 46, 1.0 / 47, 1.0 / 48, 1.0 / 49, 1.0 / 50, 1.0 / 51, 1.0 / 52, 1.0 / 53, 1.0 / 54, 1.0 / 55,
    1.0 / 56, 1.0 / 57, 1.0 / 58, 1.0 / 59, 1.0 / 60, 1.0 / 61, 1.0 / 62, 1.0 / 63, 1.0 / 64};
template <typename T>
__device__ __forceinline__ T rcp_of(int k) { return k <= kExpMaxDegree ? T(kRcp[k]) : T(1) / T(k); }

// Signature of a straight line: exp(z)_t[w] = z[w_1] ... z[w_t] / t!   (siglib/cpsig/cp_sig_join.h:36-60)
// A thread writes the words (a, rest) for FAN consecutive first letters a: the product over `rest` is shared
// (work items as in the Chen product kernels, chen_items).
template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void linear_sig_kernel(
    const T* __restrict__ disp, T* __restrict__ out, int64_t batch, DivBy<I> dv, I items, int64_t stride, int off)
{
    const I d = I(dv.d);
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* z = disp + b * int64_t(d);
        T* o = out + b * stride;
        for (I item = I(blockIdx.x) * kBlock + threadIdx.x; item < items; item += I(gridDim.x) * kBlock) {
            const FanItem<I> fi = fan_item<I, FAN>(item, d);
            T v = rcp_of<T>(fi.t);
            I idx = fi.rest;
            for (int k = fi.t - 1; k >= 1; --k) {        // letters of rest from the right
                const I q = dv.quot(idx);
                v *= z[idx - q * d] * rcp_of<T>(k);
                idx = q;
            }
#pragma unroll
            for (int i = 0; i < FAN; ++i)
                if (fi.a0 + i < d) o[off + fi.lo + (fi.a0 + i) * fi.size + fi.rest] = v * z[fi.a0 + i];
            if (off && item == 0) o[0] = T(1);
        }
    }
}

// The same rows with a level per block: a thread takes one word `rest` of t - 1 letters and writes the d words
// (a, rest): one product per d outputs, and the level, its size and its start are block-uniform (scalar arithmetic),
// where the item form above spends ~60 instructions per output on finding them per thread.  Stores stay coalesced
// (consecutive threads, consecutive `rest`).  The block keeps z in LDS (dynamic, d entries) when z_lds is set.
struct LevelBlocks {
    int top;
    uint32_t first[kExpMaxDegree + 2];      // first block of level t, t = 1 .. top; first[top + 1] = number of blocks
};
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void linear_sig_levels_kernel(
    const T* __restrict__ disp, T* __restrict__ out, int64_t batch, DivBy<I> dv, LevelBlocks lb, int64_t stride, int off,
    int z_lds)
{
    extern __shared__ double linear_lds_raw[];
    T* zl = reinterpret_cast<T*>(linear_lds_raw);
    const I d = I(dv.d);
    int t = 1;
    while (t < lb.top && blockIdx.x >= lb.first[t + 1]) ++t;
    I size = 1, lo = 0;                     // d^(t-1), start of level t
    T scale = T(1);                         // 1 / t!
    for (int k = 1; k < t; ++k) {
        lo += size * d;
        size *= d;
    }
    for (int k = 1; k <= t; ++k) scale *= rcp_of<T>(k);
    const I rest = I(blockIdx.x - lb.first[t]) * kBlock + threadIdx.x;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* z = disp + b * int64_t(d);
        if (z_lds) {
            __syncthreads();                // the row before is done with the copy
            for (I j = threadIdx.x; j < d; j += kBlock) zl[j] = z[j];
            __syncthreads();
            z = zl;
        }
        T* o = out + b * stride;
        if (rest < size) {
            T v = scale;
            I idx = rest;
            for (int k = t - 1; k >= 1; --k) {      // letters of rest from the right
                const I q = dv.quot(idx);
                v *= z[idx - q * d];
                idx = q;
            }
            T* dst = o + off + lo + rest;
            for (I a = 0; a < d; ++a) dst[a * size] = v * z[a];
        }
        if (off && blockIdx.x == 0 && threadIdx.x == 0) o[0] = T(1);
    }
}
// host: the launch of linear_sig_levels_kernel for rows of `top` levels; false when the blocks do not fit a grid
static bool level_blocks(uint64_t d, uint64_t top, LevelBlocks& lb)
{
    if (top > uint64_t(kExpMaxDegree)) return false;
    lb.top = int(top);
    uint64_t blocks = 0, size = 1;
    for (uint64_t t = 1; t <= top; ++t) {
        lb.first[t] = uint32_t(blocks);
        blocks += (size + kBlock - 1) / kBlock;
        if (blocks > 0x7fffffffull) return false;
        size *= d;
    }
    lb.first[top + 1] = uint32_t(blocks);
    return true;
}
template <typename T>
static bool launch_linear_sig_levels(const T* disp, T* out, uint64_t batch, uint64_t dimension, uint64_t top, uint64_t n_coef,
                                     int64_t stride, int off, hipStream_t stream)
{
    LevelBlocks lb;
    if (top < 1 || !level_blocks(dimension, top, lb)) return false;
    const int z_lds = dimension * sizeof(T) <= 32768;
    const dim3 grid{lb.first[top + 1], unsigned(std::min<uint64_t>(batch, 65535)), 1};
    launch_indexed(n_coef, 1, 1, [&](auto ix, dim3) {
        using I = decltype(ix);
        hipLaunchKernelGGL((linear_sig_levels_kernel<T, I>), grid, dim3(kBlock), z_lds ? size_t(dimension) * sizeof(T) : 0, stream,
                           disp, out, int64_t(batch), DivBy<I>(dimension), lb, stride, off, z_lds);
    });
    return true;
}

// out = A (x) exp(z) (append) or exp(z) (x) A (prepend):
//   append : out_t[w] = sum_{k=0..t} A_{t-k}[w_1..w_{t-k}] * z[w_{t-k+1}] ... z[w_t] / k!
//   prepend: out_t[w] = sum_{k=0..t} z[w_1] ... z[w_k] / k! * A_{t-k}[w_{k+1}..w_t]          (A_0 = 1)
// (siglib/cpsig/cp_sig_join.h:107-160).  A thread computes the words (a, rest) for FAN consecutive first letters a.
// append: the products of trailing letters are shared, the prefixes (a, head of rest) differ by d^(t-k-1) per letter;
// prepend: every term with k >= 1 carries the factor z[a] and otherwise depends on `rest` only, so
//   out_t[(a, rest)] = A_t[(a, rest)] + z[a] * C(rest),   C = sum_{k=1..t} z[r_1] .. z[r_{k-1}] / k! * A_{t-k}[r_k .. r_{t-1}].
// low_n > 0 (append form): the block keeps the first low_n coefficients of A (whole levels) and the d letters' values in
// LDS (dynamic, low_n + d entries) and reads the prefixes of those levels from there, as the Chen product kernels do.
template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void sig_join_kernel(
    const T* __restrict__ A, const T* __restrict__ disp, T* __restrict__ out, int64_t batch, DivBy<I> dv, I items,
    int64_t stride, int off, int prepend, I low_n, int z_lds)
{
    extern __shared__ double join_low_raw[];
    T* al = reinterpret_cast<T*>(join_low_raw);
    T* zl = al + low_n;
    const I d = I(dv.d);
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* a = A + b * stride + off;
        const T* z = disp + b * int64_t(d);
        if (low_n || z_lds) {       // z_lds: the letters' values alone (both forms pick them per lane)
            __syncthreads();        // the row before is done with the copies
            for (I j = threadIdx.x; j < low_n; j += kBlock) al[j] = a[j];
            for (I j = threadIdx.x; j < d; j += kBlock) zl[j] = z[j];
            __syncthreads();
            z = zl;
        }
        T* o = out + b * stride;
        for (I item = I(blockIdx.x) * kBlock + threadIdx.x; item < items; item += I(gridDim.x) * kBlock) {
            const FanItem<I> fi = fan_item<I, FAN>(item, d);
            const int t = fi.t;
            T acc[FAN];
            if (!prepend) {
#pragma unroll
                for (int i = 0; i < FAN; ++i) acc[i] = T(0);
                T ek = T(1);                       // z[w_{t-k+1}] .. z[w_t] / k!
                I head = fi.rest;                  // first t-1-k letters of rest
                I lev = fi.size * d, lo = fi.lo;   // size and start of level t-k+1 of A
                for (int k = 1; k <= t - 1; ++k) {
                    const I q = dv.quot(head);
                    ek *= z[head - q * d] * rcp_of<T>(k);
                    head = q;
                    lev = dv.quot(lev);            // d^(t-k)
                    lo -= lev;
                    const I st = dv.quot(lev);     // d^(t-k-1): distance between the prefixes of consecutive first letters
                    if (lo < low_n) {           // a whole level: the same for every lane but at level borders
                        const T* ap = al + lo + head;
#pragma unroll
                        for (int i = 0; i < FAN; ++i) {
                            const I letter = fi.a0 + i < d ? fi.a0 + i : d - 1;
                            acc[i] = fmadd(ap[letter * st], ek, acc[i]);
                        }
                    } else {
                        const T* ap = a + lo + head;
#pragma unroll
                        for (int i = 0; i < FAN; ++i) {
                            const I letter = fi.a0 + i < d ? fi.a0 + i : d - 1;
                            acc[i] = fmadd(ap[letter * st], ek, acc[i]);
                        }
                    }
                }
                // k = t: the empty prefix (A_0 = 1) and the whole word's product
                const T et = ek * rcp_of<T>(t);
#pragma unroll
                for (int i = 0; i < FAN; ++i) {
                    const I letter = fi.a0 + i < d ? fi.a0 + i : d - 1;
                    acc[i] = fmadd(et, z[letter], acc[i]);
                }
            } else {
                // letters of rest from the left: reverse it once (the divisions deliver letters right to left)
                I idx = fi.rest, rev = 0;
                for (int k = 0; k < t - 1; ++k) {
                    const I q = dv.quot(idx);
                    rev = rev * d + (idx - q * d);
                    idx = q;
                }
                // C = sum_{k=1..t} P_{k-1} / k! * A_{t-k}[suffix], P_j = z[r_1] .. z[r_j]
                T c = T(0);
                T pk = T(1);                       // P_{k-1} / k!
                I rem = fi.rest, size = fi.size, lo = fi.lo;      // suffix r_k .. r_{t-1}, d^(t-k), start of level t-k+1
                for (int k = 1; k <= t; ++k) {
                    pk *= rcp_of<T>(k);
                    lo -= size;                    // start of level t-k
                    c = fmadd(k < t ? a[lo + rem] : T(1), pk, c);
                    if (k < t) {
                        const I q = dv.quot(rev);
                        const I letter = rev - q * d;          // r_k
                        rev = q;
                        size = dv.quot(size);                  // d^(t-k-1)
                        pk *= z[letter];
                        rem -= letter * size;
                    }
                }
#pragma unroll
                for (int i = 0; i < FAN; ++i) {
                    const I letter = fi.a0 + i < d ? fi.a0 + i : d - 1;
                    acc[i] = z[letter] * c;
                }
            }
#pragma unroll
            for (int i = 0; i < FAN; ++i) {
                if (fi.a0 + i < d) {
                    const I r = fi.lo + (fi.a0 + i) * fi.size + fi.rest;
                    o[off + r] = a[r] + acc[i];
                }
            }
            if (off && item == 0) o[0] = T(1);
        }
    }
}

// Adjoint of z -> exp(z): dz[j] = sum_t 1/t! sum_{w in d^t} dE_t[w] sum_{i : w_i = j} prod_{m != i} z[w_m]
// (closed form of the level recursion in siglib/cpsig/cp_sig_combine.h:232-263).  A thread takes the words (a, rest)
// for FAN consecutive first letters a (work items as in the Chen product kernels): the first position gives
// dz[a] += dE[(a, rest)] * prod(rest) / t!, and for a letter r_i of `rest` the terms of all a collapse into
// dz[r_i] += (sum_a z[a] dE[(a, rest)]) * prod_{m != i} z[r_m] / t!  - FAN + t - 1 additions instead of FAN * t.
// The letters and suffix products of `rest` sit in arrays of TMAX entries that every loop walks with compile-time
// bounds, so that they stay in registers (TMAX >= degree - 1; 64: rolled loops, arrays in scratch memory).
// Per-block partial sums in LDS (or straight to HBM for very wide paths), dz zeroed beforehand.
constexpr int kExpAccMax = 4096;
template <typename T, typename I, int FAN, int TMAX>
__global__ __launch_bounds__(kBlock) void exp_pullback_kernel(
    const T* __restrict__ dE, const T* __restrict__ disp, T* __restrict__ dz, int64_t batch, DivBy<I> dv, I items,
    int64_t stride, int off, int use_lds, int copies)
{
    extern __shared__ double exp_lds_raw[];
    T* acc = reinterpret_cast<T*>(exp_lds_raw);
    const I d = I(dv.d);
    // `copies` private sets of d accumulators, chosen by lane: few letters mean many lanes adding to one word
    T* mine = acc + (threadIdx.x % copies) * d;
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        const T* z = disp + b * int64_t(d);
        if (use_lds) {
            // the accumulators and, behind them, the row's d letter values (picked per lane: from memory every such
            // load would occupy the texture addresser for a whole wave)
            T* zl = acc + I(copies) * d;
            __syncthreads();
            for (I j = threadIdx.x; j < I(copies) * d; j += kBlock) acc[j] = T(0);
            for (I j = threadIdx.x; j < d; j += kBlock) zl[j] = z[j];
            __syncthreads();
            z = zl;
        }
        const T* g = dE + b * stride + off;
        T* out = dz + b * int64_t(d);
        auto add = [&](I letter, T v) {
            if (use_lds) lds_add_shared(&mine[letter], v);
            else dev_add(&out[letter], v);
        };
        for (I item = I(xcd_block_2d().x) * kBlock + threadIdx.x; item < items; item += I(gridDim.x) * kBlock) {
            const FanItem<I> fi = fan_item<I, FAN>(item, d);
            const int n = fi.t - 1;         // letters of rest
            T suf[TMAX];                    // suf[i] = z[r_{i+1}] .. z[r_{n-1}] / t!   (0-based position i in rest)
            I let[TMAX];
            T run = T(1);
            for (int k = 1; k <= fi.t; ++k) run *= rcp_of<T>(k);
            I idx = fi.rest;
            if constexpr (TMAX < 64) {
#pragma unroll
                for (int i = TMAX - 1; i >= 0; --i) {
                    if (i < n) {
                        const I q = dv.quot(idx);
                        let[i] = idx - q * d;
                        idx = q;
                        suf[i] = run;
                        run *= z[let[i]];
                    }
                }
            } else {
                for (int i = n - 1; i >= 0; --i) {
                    const I q = dv.quot(idx);
                    let[i] = idx - q * d;
                    idx = q;
                    suf[i] = run;
                    run *= z[let[i]];
                }
            }
            // run = prod(rest) / t!
            T wsum = T(0);
#pragma unroll
            for (int i = 0; i < FAN; ++i) {
                if (fi.a0 + i < d) {
                    const T e = g[fi.lo + (fi.a0 + i) * fi.size + fi.rest];
                    add(fi.a0 + i, e * run);
                    wsum = fmadd(z[fi.a0 + i], e, wsum);
                }
            }
            T pre = wsum;                   // wsum * z[r_0] .. z[r_{i-1}]
            if constexpr (TMAX < 64) {
#pragma unroll
                for (int i = 0; i < TMAX; ++i) {
                    if (i < n) {
                        add(let[i], pre * suf[i]);
                        pre *= z[let[i]];
                    }
                }
            } else {
                for (int i = 0; i < n; ++i) {
                    add(let[i], pre * suf[i]);
                    pre *= z[let[i]];
                }
            }
        }
        if (use_lds) {
            // the private sets fold into the first one with the whole block at work (d lanes walking them one read at
            // a time would take longer than the block's items), then one atomic per letter
            __syncthreads();
            for (I e = d + threadIdx.x; e < I(copies) * d; e += kBlock) lds_add_shared(&acc[e % d], acc[e]);
            __syncthreads();
            for (I j = threadIdx.x; j < d; j += kBlock) dev_add(&out[j], acc[j]);
        }
    }
}

// d = 1: exp(z)_k = z^k / k!, so dz = sum_k dE_k z^(k-1) / (k-1)!
template <typename T>
__global__ __launch_bounds__(kBlock) void exp_pullback_dim_one_kernel(
    const T* __restrict__ dE, const T* __restrict__ disp, T* __restrict__ dz, int64_t batch, int64_t degree, int64_t stride, int off)
{
    for (int64_t b = int64_t(blockIdx.x) * kBlock + threadIdx.x; b < batch; b += int64_t(gridDim.x) * kBlock) {
        const T z = disp[b];
        const T* g = dE + b * stride + off;
        T pw = T(1), sum = T(0);
        for (int64_t k = 1; k <= degree; ++k) {
            sum = fmadd(g[k - 1], pw, sum);
            pw *= z / T(k);
        }
        dz[b] = sum;
    }
}

template <typename T>
static void sig_combine_impl(const T* sig1, const T* sig2, T* out, uint64_t batch, uint64_t dimension, uint64_t degree,
                             bool scalar_term)
{
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_combine_cuda");
    if (batch == 0) return;
    checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {        // degree 0: only the scalar slot exists
        if (scalar_term)
            hipLaunchKernelGGL((fill_trivial_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch),
                               int64_t(1), 1);
    } else {
        with_chen_fan(dimension, [&](auto fan) {
            constexpr int FAN = decltype(fan)::value;
            const uint64_t items = chen_items(dimension, degree, FAN);
            // the short levels of both factors in LDS; a thread then takes several items, so that the copy is amortised
            const uint64_t blocks = (items + kBlock - 1) / kBlock * batch;
            const uint64_t low_n = chen_low_count(dimension, degree, sizeof(T), blocks);
            const uint64_t per_thread = low_n ? chen_low_items_per_thread(low_n, blocks) : 1;
            launch_indexed(s.n_coef, (items + per_thread - 1) / per_thread, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                hipLaunchKernelGGL((sig_combine_kernel<T, I, FAN>), grid, dim3(kBlock), 2 * low_n * sizeof(T), stream, sig1, sig2, out,
                                   int64_t(batch), DivBy<I>(dimension), I(items), int64_t(s.stride), int64_t(s.stride),
                                   int64_t(s.stride), s.off, s.off, s.off, I(low_n));
            });
        });
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void sig_combine_backprop_impl(const T* derivs, T* d1, T* d2, const T* sig1, const T* sig2, uint64_t batch,
                                      uint64_t dimension, uint64_t degree, bool scalar_term)
{
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_combine_backprop_cuda");
    if (batch == 0) return;
    checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term) {
            hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, d1, int64_t(batch));
            hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, d2, int64_t(batch));
        }
    } else {
        launch_combine_bwd<T>(derivs, d1, d2, sig1, sig2, batch, dimension, degree, s, stream);
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}


template <typename T>
static void linear_sig_impl(const T* disp, T* out, uint64_t batch, uint64_t dimension, uint64_t degree, bool scalar_term)
{
    const SigShape s = sig_shape(dimension, degree, scalar_term, "linear_sig_cuda");
    if (batch == 0) return;
    checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term)
            hipLaunchKernelGGL((fill_trivial_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch),
                               int64_t(1), 1);
    } else {
        if (!launch_linear_sig_levels<T>(disp, out, batch, dimension, degree, s.n_coef, int64_t(s.stride), s.off, stream))
            with_chen_fan(dimension, [&](auto fan) {
                constexpr int FAN = decltype(fan)::value;
                const uint64_t items = chen_items(dimension, degree, FAN);
                launch_indexed(s.n_coef, items, batch, [&](auto ix, dim3 grid) {
                    using I = decltype(ix);
                    hipLaunchKernelGGL((linear_sig_kernel<T, I, FAN>), grid, dim3(kBlock), 0, stream, disp, out, int64_t(batch),
                                       DivBy<I>(dimension), I(items), int64_t(s.stride), s.off);
                });
            });
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void sig_join_impl(const T* sig, const T* disp, T* out, uint64_t batch, uint64_t dimension, uint64_t degree,
                          bool prepend, bool scalar_term)
{
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_join_cuda");
    if (batch == 0) return;
    checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term)
            hipLaunchKernelGGL((fill_trivial_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch),
                               int64_t(1), 1);
    } else {
        with_chen_fan(dimension, [&](auto fan) {
            constexpr int FAN = decltype(fan)::value;
            const uint64_t items = chen_items(dimension, degree, FAN);
            const uint64_t blocks = (items + kBlock - 1) / kBlock * batch;
            const uint64_t low_n = prepend ? 0 : chen_low_count(dimension, degree, sizeof(T), blocks);
            const uint64_t per_thread = low_n ? chen_low_items_per_thread(low_n, blocks) : 1;
            launch_indexed(s.n_coef, (items + per_thread - 1) / per_thread, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                const int z_lds = dimension * sizeof(T) <= 32768;
                hipLaunchKernelGGL((sig_join_kernel<T, I, FAN>), grid, dim3(kBlock),
                                   (low_n || z_lds) ? (low_n + dimension) * sizeof(T) : 0, stream, sig, disp, out, int64_t(batch),
                                   DivBy<I>(dimension), I(items), int64_t(s.stride), s.off, int(prepend), I(low_n), z_lds);
            });
        });
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void sig_join_backprop_impl(const T* d_out, T* d_sig, T* d_disp, const T* sig, const T* disp, uint64_t batch,
                                   uint64_t dimension, uint64_t degree, bool prepend, bool scalar_term)
{
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_join_backprop_cuda");
    if (batch == 0) return;
    const uint64_t bytes = checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    const uint64_t dz_elems = checked_mul(batch, dimension, "displacement gradient");
    if (dimension >= 2 && degree >= uint64_t(kExpMaxDegree)) throw std::runtime_error("sig_join_backprop_cuda: degree too high");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(dz_elems)), dim3(kBlock), 0, stream, d_disp, int64_t(dz_elems));
    if (s.n_coef == 0) {
        if (scalar_term) hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, d_sig, int64_t(batch));
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    T* E = static_cast<T*>(workspace(4, bytes));
    T* dE = static_cast<T*>(workspace(5, bytes));
    // exp(z) up to level degree - 1: the adjoint never multiplies with a factor's top level
    if (degree >= 2 && !launch_linear_sig_levels<T>(disp, E, batch, dimension, degree - 1, s.n_coef, int64_t(s.stride), s.off, stream))
        with_chen_fan(dimension, [&](auto fan) {
            constexpr int FAN = decltype(fan)::value;
            const uint64_t items = chen_items(dimension, degree - 1, FAN);
            launch_indexed(s.n_coef, items, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                hipLaunchKernelGGL((linear_sig_kernel<T, I, FAN>), grid, dim3(kBlock), 0, stream, disp, E, int64_t(batch),
                                   DivBy<I>(dimension), I(items), int64_t(s.stride), s.off);
            });
        });
    // the Chen product's adjoint with exp(z) as the right (append) or left (prepend) factor; as the right factor its
    // kernel may fold the levels above `top` into d_disp, and the adjoint of exp below then stops at `top`
    ExpFold<T> fold;
    fold.z = disp;
    fold.dz = d_disp;
    fold.level = int(degree);
    if (prepend) launch_combine_bwd<T>(d_out, dE, d_sig, (const T*)E, sig, batch, dimension, degree, s, stream);
    else launch_combine_bwd<T>(d_out, d_sig, dE, sig, (const T*)E, batch, dimension, degree, s, stream, 3, SharedRows(), 2, &fold);
    const uint64_t top = uint64_t(fold.level);
    if (dimension == 1) {
        hipLaunchKernelGGL((exp_pullback_dim_one_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, (const T*)dE, disp,
                           d_disp, int64_t(batch), int64_t(degree), int64_t(s.stride), s.off);
    } else {
        const int use_lds = dimension <= uint64_t(kExpAccMax);
        const int copies = use_lds ? int(std::max<uint64_t>(1, std::min<uint64_t>(32, uint64_t(kExpAccMax) / dimension))) : 1;
        with_chen_fan(dimension, [&](auto fan) {
            constexpr int FAN = decltype(fan)::value;
            const uint64_t items = chen_items(dimension, top, FAN);
            // a few items per thread, so that a block's LDS partial sums amortise their flush
            launch_indexed(s.n_coef, (items + 3) / 4, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                auto go = [&](auto tmax) {
                    constexpr int TMAX = decltype(tmax)::value;
                    hipLaunchKernelGGL((exp_pullback_kernel<T, I, FAN, TMAX>), grid, dim3(kBlock),
                                       use_lds ? (size_t(copies) + 1) * size_t(dimension) * sizeof(T) : 0, stream, (const T*)dE, disp,
                                       d_disp, int64_t(batch), DivBy<I>(dimension), I(items), int64_t(s.stride), s.off, use_lds,
                                       copies);
                };
                if (top <= 5) go(IntC<4>{});
                else if (top <= 9) go(IntC<8>{});
                else if (top <= 17) go(IntC<16>{});
                else go(IntC<64>{});
            });
        });
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

static void path_shape_check(uint64_t dimension, uint64_t length, const char* who)
{
    if (dimension == 0) throw std::invalid_argument(std::string(who) + " received path of dimension 0");
    if (dimension > 0x3fffffff || length > (uint64_t(1) << 40)) throw std::invalid_argument(std::string(who) + ": shape out of range");
}

template <typename T>
static void transform_path_impl(const T* in, T* out, uint64_t batch, uint64_t dimension, uint64_t length, bool time_aug,
                                bool lead_lag, T end_time)
{
    path_shape_check(dimension, length, "transform_path_cuda");
    if (batch == 0 || length == 0) return;
    const uint64_t td = (lead_lag ? 2 * dimension : dimension) + (time_aug ? 1 : 0);
    const uint64_t tl = lead_lag ? 2 * length - 1 : length;
    const uint64_t total = checked_mul(checked_mul(batch, tl, "transformed path"), td, "transformed path");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    const T scale = tl > 1 ? end_time / T(tl - 1) : T(0);
    (void)total;
    launch_indexed(tl * td, (tl * td + kTransformBatch - 1) / kTransformBatch, batch, [&](auto ix, dim3 grid) {
        using I = decltype(ix);
        hipLaunchKernelGGL((transform_path_kernel<T, I>), grid, dim3(kBlock), 0, stream, in, out, int64_t(batch), I(length),
                           I(dimension), DivBy<I>(td), int(time_aug), int(lead_lag), scale);
    });
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void transform_path_backprop_impl(const T* derivs, T* out, uint64_t batch, uint64_t dimension, uint64_t length,
                                         bool time_aug, bool lead_lag)
{
    path_shape_check(dimension, length, "transform_path_backprop_cuda");
    if (batch == 0 || length == 0) return;
    const uint64_t total = checked_mul(checked_mul(batch, length, "path gradient"), dimension, "path gradient");
    SIG_HIP(hipDeviceSynchronize());
    hipStream_t stream = nullptr;
    (void)total;
    const uint64_t td = (lead_lag ? 2 * dimension : dimension) + (time_aug ? 1 : 0);
    const uint64_t tl = lead_lag ? 2 * length - 1 : length;
    checked_mul(checked_mul(batch, tl, "transformed path"), td, "transformed path");
    launch_indexed(tl * td, length * dimension, batch, [&](auto ix, dim3 grid) {
        using I = decltype(ix);
        hipLaunchKernelGGL((transform_path_bwd_kernel<T, I>), grid, dim3(kBlock), 0, stream, derivs, out, int64_t(batch),
                           I(length), DivBy<I>(dimension), int(time_aug), int(lead_lag));
    });
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

}  // namespace sigamd

using namespace sigamd;

extern "C" {

CUSIG_AMD_API int sig_combine_cuda_f(const float* sig1, const float* sig2, float* out, uint64_t batch_size,
                                     uint64_t dimension, uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] { sig_combine_impl<float>(sig1, sig2, out, batch_size, dimension, degree, scalar_term); });
}
CUSIG_AMD_API int sig_combine_cuda_d(const double* sig1, const double* sig2, double* out, uint64_t batch_size,
                                     uint64_t dimension, uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] { sig_combine_impl<double>(sig1, sig2, out, batch_size, dimension, degree, scalar_term); });
}
CUSIG_AMD_API int sig_combine_backprop_cuda_f(const float* sig_combined_deriv, float* sig1_deriv, float* sig2_deriv,
                                              const float* sig1, const float* sig2, uint64_t batch_size,
                                              uint64_t dimension, uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] {
        sig_combine_backprop_impl<float>(sig_combined_deriv, sig1_deriv, sig2_deriv, sig1, sig2, batch_size, dimension,
                                         degree, scalar_term);
    });
}
CUSIG_AMD_API int sig_combine_backprop_cuda_d(const double* sig_combined_deriv, double* sig1_deriv, double* sig2_deriv,
                                              const double* sig1, const double* sig2, uint64_t batch_size,
                                              uint64_t dimension, uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] {
        sig_combine_backprop_impl<double>(sig_combined_deriv, sig1_deriv, sig2_deriv, sig1, sig2, batch_size, dimension,
                                          degree, scalar_term);
    });
}
CUSIG_AMD_API int transform_path_cuda_f(const float* data_in, float* data_out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t length, bool time_aug, bool lead_lag, float end_time) noexcept
{
    return guarded([&] { transform_path_impl<float>(data_in, data_out, batch_size, dimension, length, time_aug, lead_lag, end_time); });
}
CUSIG_AMD_API int transform_path_cuda_d(const double* data_in, double* data_out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t length, bool time_aug, bool lead_lag, double end_time) noexcept
{
    return guarded([&] { transform_path_impl<double>(data_in, data_out, batch_size, dimension, length, time_aug, lead_lag, end_time); });
}
CUSIG_AMD_API int transform_path_backprop_cuda_f(const float* derivs, float* data_out, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t length, bool time_aug, bool lead_lag,
                                                 float) noexcept
{
    return guarded([&] { transform_path_backprop_impl<float>(derivs, data_out, batch_size, dimension, length, time_aug, lead_lag); });
}
CUSIG_AMD_API int transform_path_backprop_cuda_d(const double* derivs, double* data_out, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t length, bool time_aug, bool lead_lag,
                                                 double) noexcept
{
    return guarded([&] { transform_path_backprop_impl<double>(derivs, data_out, batch_size, dimension, length, time_aug, lead_lag); });
}

CUSIG_AMD_API int linear_sig_cuda_f(const float* displacement, float* out, uint64_t batch_size, uint64_t dimension,
                                    uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] { linear_sig_impl<float>(displacement, out, batch_size, dimension, degree, scalar_term); });
}
CUSIG_AMD_API int linear_sig_cuda_d(const double* displacement, double* out, uint64_t batch_size, uint64_t dimension,
                                    uint64_t degree, bool scalar_term) noexcept
{
    return guarded([&] { linear_sig_impl<double>(displacement, out, batch_size, dimension, degree, scalar_term); });
}
CUSIG_AMD_API int sig_join_cuda_f(const float* sig, const float* displacement, float* out, uint64_t batch_size,
                                  uint64_t dimension, uint64_t degree, bool prepend, bool scalar_term) noexcept
{
    return guarded([&] { sig_join_impl<float>(sig, displacement, out, batch_size, dimension, degree, prepend, scalar_term); });
}
CUSIG_AMD_API int sig_join_cuda_d(const double* sig, const double* displacement, double* out, uint64_t batch_size,
                                  uint64_t dimension, uint64_t degree, bool prepend, bool scalar_term) noexcept
{
    return guarded([&] { sig_join_impl<double>(sig, displacement, out, batch_size, dimension, degree, prepend, scalar_term); });
}
CUSIG_AMD_API int sig_join_backprop_cuda_f(const float* d_out, float* d_sig, float* d_displacement, const float* sig,
                                           const float* displacement, uint64_t batch_size, uint64_t dimension,
                                           uint64_t degree, bool prepend, bool scalar_term) noexcept
{
    return guarded([&] {
        split_on_bad_alloc(batch_size, "sig_join_backprop", [&](uint64_t first, uint64_t count) {
            const uint64_t stride = first ? sig_shape(dimension, degree, scalar_term, "sig_join_backprop_cuda").stride : 0;
            sig_join_backprop_impl<float>(d_out + first * stride, d_sig + first * stride, d_displacement + first * dimension,
                                      sig + first * stride, displacement + first * dimension, count, dimension, degree, prepend,
                                      scalar_term);
        });
    });
}
CUSIG_AMD_API int sig_join_backprop_cuda_d(const double* d_out, double* d_sig, double* d_displacement, const double* sig,
                                           const double* displacement, uint64_t batch_size, uint64_t dimension,
                                           uint64_t degree, bool prepend, bool scalar_term) noexcept
{
    return guarded([&] {
        split_on_bad_alloc(batch_size, "sig_join_backprop", [&](uint64_t first, uint64_t count) {
            const uint64_t stride = first ? sig_shape(dimension, degree, scalar_term, "sig_join_backprop_cuda").stride : 0;
            sig_join_backprop_impl<double>(d_out + first * stride, d_sig + first * stride, d_displacement + first * dimension,
                                       sig + first * stride, displacement + first * dimension, count, dimension, degree, prepend,
                                       scalar_term);
        });
    });
}

}  // extern "C"
