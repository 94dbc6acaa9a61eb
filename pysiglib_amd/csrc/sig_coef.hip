// Coefficients of selected words and their backward pass, behind the reference's entry points
//   sig_coef_cuda_{f,d}, sig_coef_backprop_cuda_{f,d}   (decl siglib/cusig/cusig.h:450-494; arithmetic of
//   siglib/cpsig/cp_sig_coef_impl.cpp:35-84,296-305 forward and :360-485 backward).
// One lane sweeps the path for one (path, word) pair and keeps the word's prefix coefficients in registers: the
// per-word Horner chain is the prefix chain of the signature sweep without a subtree below it.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "../../include/cusig_amd.h"
#include "sig_host.h"
#include "sig_kernels.h"

namespace sigamd {

constexpr int kCoefMaxDegree = 64;
// 1/i!, i = 0 .. 64, rounded the way the reference builds its table (each entry the previous one divided by i,
// siglib/cpsig/cp_sig_coef_impl.cpp:186-191)
__constant__ double kInvFact[kCoefMaxDegree + 1] = {
    1.0, 1.0, 0.5, 0.16666666666666666, 0.041666666666666664, 0.008333333333333333, 0.001388888888888889,
    0.0001984126984126984, 2.48015873015873e-05, 2.7557319223985893e-06, 2.7557319223985894e-07,
    2.505210838544172e-08, 2.08767569878681e-09, 1.6059043836821616e-10, 1.1470745597729726e-11,
    7.647163731819817e-13, 4.779477332387386e-14, 2.811457254345521e-15, 1.5619206968586228e-16,
    8.220635246624331e-18, 4.1103176233121653e-19, 1.9572941063391263e-20, 8.896791392450574e-22,
    3.868170170630684e-23, 1.6117375710961184e-24, 6.446950284384474e-26, 2.4795962632247976e-27,
    9.183689863795547e-29, 3.2798892370698385e-30, 1.1309962886447718e-31, 3.769987628815906e-33,
    1.2161250415535181e-34, 3.800390754854744e-36, 1.151633562077195e-37, 3.387157535521162e-39,
    9.67759295863189e-41, 2.6882202662866363e-42, 7.265460179153071e-44, 1.911963205040282e-45,
    4.902469756513544e-47, 1.2256174391283858e-48, 2.9893108271424046e-50, 7.117406731291439e-52,
    1.6552108677421951e-53, 3.7618428812322616e-55, 8.359650847182803e-57, 1.817315401561479e-58,
    3.8666285139605935e-60, 8.055476070751236e-62, 1.6439747083165788e-63, 3.2879494166331576e-65,
    6.446959640457172e-67, 1.2397999308571486e-68, 2.3392451525606576e-70, 4.3319354677049213e-72,
    7.876246304918039e-74, 1.4064725544496498e-75, 2.467495709560789e-77, 4.2543029475186016e-79,
    7.210682961895935e-81, 1.2017804936493225e-82, 1.970131956802168e-84, 3.1776321883905935e-86,
    5.043860616493006e-88, 7.881032213270321e-90};

struct WordList {
    const uint64_t* letters;     // all words end to end
    const uint64_t* start;       // first letter of word w
    const uint64_t* out_start;   // first output column of word w
    const uint64_t* degree;
    uint64_t count;
};

// c_i += z_{i-1} * (((1/i!) z_0 + c_1/(i-1)!) z_1 + ... + c_{i-1}/1!),  i = k .. 1  (descending: every read of a
// shorter prefix still sees the value from before the step).  SIGN = -1 applies exp(-z) instead of exp(z).
// UF: unroll factor of every loop over letters (KMAX + 1 = fully unrolled, the arrays live in registers; 1 = rolled
// loops over arrays in scratch memory, for long words).
template <typename T, int KMAX, int UF, int SIGN>
__device__ __forceinline__ void word_step(T (&c)[KMAX + 1], const T (&z)[KMAX], int k)
{
#pragma unroll UF
    for (int i = KMAX; i >= 1; --i) {
        if (i <= k) {
            T acc = T((SIGN < 0 && (i & 1)) ? -kInvFact[i] : kInvFact[i]);
#pragma unroll UF
            for (int j = 0; j + 1 < i; ++j) {
                const int m = i - j - 1;
                acc = fmadd(acc, z[j], c[j + 1] * T((SIGN < 0 && (m & 1)) ? -kInvFact[m] : kInvFact[m]));
            }
            c[i] = fmadd(acc, z[i - 1], c[i]);
        }
    }
}

template <typename T, int KMAX, int UF>
__global__ __launch_bounds__(kBlock) void sig_coef_kernel(
    const T* __restrict__ path, T* __restrict__ out, WordList words, int64_t batch, int64_t d, int64_t len, int64_t row,
    int prefixes)
{
    const int64_t total = batch * int64_t(words.count);
    for (int64_t item = int64_t(blockIdx.x) * kBlock + threadIdx.x; item < total; item += int64_t(gridDim.x) * kBlock) {
        const int64_t b = item / int64_t(words.count), w = item % int64_t(words.count);
        const int k = int(words.degree[w]);
        T* o = out + b * row + (prefixes ? int64_t(words.out_start[w]) : w);
        if (k == 0) { o[0] = T(1); continue; }
        if (k > KMAX) continue;     // the host picks KMAX >= the largest degree
        int64_t let[KMAX];
        T c[KMAX + 1], z[KMAX], prev[KMAX];
        const T* x = path + b * len * d;
#pragma unroll UF
        for (int i = 0; i < KMAX; ++i) {
            let[i] = i < k ? int64_t(words.letters[words.start[w] + i]) : 0;
            prev[i] = len > 0 ? x[let[i]] : T(0);
            c[i + 1] = T(0);
        }
        c[0] = T(1);
        for (int64_t s = 1; s < len; ++s) {
            const T* xs = x + s * d;
#pragma unroll UF
            for (int i = 0; i < KMAX; ++i) {
                const T cur = xs[let[i]];
                z[i] = cur - prev[i];
                prev[i] = cur;
            }
            word_step<T, KMAX, UF, 1>(c, z, k);
        }
        if (prefixes) {
#pragma unroll UF
            for (int i = 1; i <= KMAX; ++i)
                if (i <= k) o[i - 1] = c[i];
        } else {
            T last = c[1];
#pragma unroll UF
            for (int i = 2; i <= KMAX; ++i)
                if (i == k) last = c[i];
            o[0] = last;
        }
    }
}

// The same sweep with the path's points staged through LDS: a block serves up to 256 words of ONE path and copies
// `chunk` points at a time with coalesced loads; the lanes then pick their letters' channels from LDS, the points of
// kCoefAhead steps at a time.  (Picked straight from memory, every lane-indexed load occupies the texture addresser
// for a whole wave whatever it coalesces to: 4 such loads per step were 61 % of a wave's cycles.)
constexpr int kCoefAhead = 4;
template <typename T, int KMAX, int UF>
__global__ __launch_bounds__(kBlock) void sig_coef_staged_kernel(
    const T* __restrict__ path, T* __restrict__ out, WordList words, int64_t batch, int64_t d, int64_t len, int64_t row,
    int prefixes, int chunk)
{
    extern __shared__ double coef_rows_raw[];
    T* rows = reinterpret_cast<T*>(coef_rows_raw);      // [chunk][d]
    const int64_t w = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const bool live = w < int64_t(words.count);
    const int k = live ? int(words.degree[w]) : 0;
    const bool active = k > 0 && k <= KMAX;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = path + b * len * d;
        int lo[KMAX];                                   // the letters as offsets into a row
        T c[KMAX + 1], z[KMAX], prev[KMAX];
#pragma unroll UF
        for (int i = 0; i < KMAX; ++i) {
            lo[i] = (active && i < k) ? int(words.letters[words.start[w] + i]) : 0;
            prev[i] = len > 0 ? x[lo[i]] : T(0);
            c[i + 1] = T(0);
        }
        c[0] = T(1);
        for (int64_t s0 = 1; s0 < len; s0 += chunk) {
            const int n = int(len - s0 < chunk ? len - s0 : chunk);
            __syncthreads();                            // the chunk before has been consumed
            for (int64_t e = threadIdx.x; e < int64_t(n) * d; e += blockDim.x) rows[e] = x[s0 * d + e];
            __syncthreads();
            if (active) {
                int r = 0;
                if constexpr (UF > 1) {
                    for (; r + kCoefAhead <= n; r += kCoefAhead) {
                        T cur[kCoefAhead][KMAX];
#pragma unroll
                        for (int u = 0; u < kCoefAhead; ++u) {
#pragma unroll
                            for (int i = 0; i < KMAX; ++i) cur[u][i] = rows[int64_t(r + u) * d + lo[i]];
                        }
#pragma unroll
                        for (int u = 0; u < kCoefAhead; ++u) {
#pragma unroll
                            for (int i = 0; i < KMAX; ++i) {
                                z[i] = cur[u][i] - prev[i];
                                prev[i] = cur[u][i];
                            }
                            word_step<T, KMAX, UF, 1>(c, z, k);
                        }
                    }
                }
                for (; r < n; ++r) {
#pragma unroll UF
                    for (int i = 0; i < KMAX; ++i) {
                        const T cur = rows[int64_t(r) * d + lo[i]];
                        z[i] = cur - prev[i];
                        prev[i] = cur;
                    }
                    word_step<T, KMAX, UF, 1>(c, z, k);
                }
            }
        }
        if (!live) continue;
        T* o = out + b * row + (prefixes ? int64_t(words.out_start[w]) : w);
        if (k == 0) { o[0] = T(1); continue; }
        if (!active) continue;
        if (prefixes) {
#pragma unroll UF
            for (int i = 1; i <= KMAX; ++i)
                if (i <= k) o[i - 1] = c[i];
        } else {
            T last = c[1];
#pragma unroll UF
            for (int i = 2; i <= KMAX; ++i)
                if (i == k) last = c[i];
            o[0] = last;
        }
    }
}

// Reverse sweep of one (path, word) pair: coefficients before the step by exp(-z), then the adjoint of the step:
// with st_j = ((1/i!) z_0 + c_1/(i-1)!) z_1 + ... (the Horner values of prefix length i),
//   dz_{i-1} += g_i st_{i-1};  walking j = i-2 .. 0 with sd = g_i z_{i-1} z_{i-2} ..:  dz_j += sd st_j,
//   g_{j+1} += sd / (i-j-1)!.
// A block serves the words blockIdx.x * blockDim.x .. of ONE path.  Its lanes add their increment gradients into
// per-step, per-channel LDS sums for a chunk of `chunk` steps (`copies` private sets per step, chosen by lane, because
// few channels mean many lanes per word of LDS); after the chunk, point p receives G(step p) - G(step p + 1) in one
// atomic per (block, point, channel), G being zero outside the chunk.  (A flush after every step had the whole block
// wait at a barrier while d lanes walked the private sets one LDS read at a time: 4400 cycles a step.)
// use_lds = 0 (very wide paths): every lane adds straight to HBM.  `out` is zeroed beforehand.
template <typename T, int KMAX, int UF>
__global__ __launch_bounds__(kBlock) void sig_coef_bwd_kernel(
    const T* __restrict__ path, T* __restrict__ out, const T* __restrict__ coefs, const T* __restrict__ derivs,
    WordList words, int64_t batch, int64_t d, int64_t len, int64_t row, int use_lds, int copies, int chunk)
{
    extern __shared__ double coef_lds_raw[];
    T* acc = reinterpret_cast<T*>(coef_lds_raw);        // [chunk][copies][d]
    T* rows = acc + int64_t(chunk) * copies * d;        // use_lds: the points s_lo - 1 .. s_hi of the chunk, [chunk + 1][d]
    const int64_t w = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
    const bool live = w < int64_t(words.count);
    const int k = live ? int(words.degree[w]) : 0;
    const bool active = k > 0 && k <= KMAX;
    const int64_t slab = int64_t(copies) * d;           // LDS entries of one step
    T* mine = acc + int64_t(threadIdx.x % copies) * d;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        int64_t let[KMAX];
        T c[KMAX + 1], g[KMAX + 1], z[KMAX], next[KMAX], st[KMAX], dz[KMAX];
        const T* x = path + b * len * d;
        T* gx = out + b * len * d;
        c[0] = T(1);
        g[0] = T(0);
        if (active) {
            const T* crow = coefs + b * row + int64_t(words.out_start[w]);
            const T* grow = derivs + b * row + int64_t(words.out_start[w]);
#pragma unroll UF
            for (int i = 0; i < KMAX; ++i) {
                let[i] = i < k ? int64_t(words.letters[words.start[w] + i]) : 0;
                next[i] = x[(len - 1) * d + let[i]];
                c[i + 1] = i < k ? crow[i] : T(0);
                g[i + 1] = i < k ? grow[i] : T(0);
            }
        }
        // copies the points of the chunk ending at step s_hi to LDS (coalesced; lane-indexed loads from memory occupy
        // the texture addresser for a whole wave each)
        auto stage = [&](int64_t s_hi) {
            const int64_t s_lo = s_hi - chunk + 1 > 1 ? s_hi - chunk + 1 : 1;
            const int64_t cnt = (s_hi - s_lo + 2) * d;
            for (int64_t e = threadIdx.x; e < cnt; e += blockDim.x) rows[e] = x[(s_lo - 1) * d + e];
        };
        if (use_lds) {
            __syncthreads();        // the previous path's sums and points have been consumed
            for (int64_t j = threadIdx.x; j < int64_t(chunk) * slab; j += blockDim.x) acc[j] = T(0);
            if (len >= 2) stage(len - 1);
            __syncthreads();
        }
        for (int64_t s_hi = len - 1; s_hi >= 1; s_hi -= chunk) {        // steps s_lo .. s_hi, downwards
            const int64_t s_lo = s_hi - chunk + 1 > 1 ? s_hi - chunk + 1 : 1;
            if (active) {
                for (int64_t s = s_hi; s >= s_lo; --s) {                // step s-1 -> s
                    const T* xp = use_lds ? rows + (s - s_lo) * d : x + (s - 1) * d;
#pragma unroll UF
                    for (int i = 0; i < KMAX; ++i) {
                        const T cur = xp[let[i]];
                        z[i] = next[i] - cur;
                        next[i] = cur;
                    }
                    word_step<T, KMAX, UF, -1>(c, z, k);
#pragma unroll UF
                    for (int i = 0; i < KMAX; ++i) dz[i] = T(0);
#pragma unroll UF
                    for (int i = 1; i <= KMAX; ++i) {
                        if (i <= k) {
                            st[0] = T(kInvFact[i]);
#pragma unroll UF
                            for (int j = 0; j + 1 < i; ++j) st[j + 1] = fmadd(st[j], z[j], c[j + 1] * T(kInvFact[i - j - 1]));
                            const T gi = g[i];
                            dz[i - 1] = fmadd(gi, st[i - 1], dz[i - 1]);
                            T sd = gi * z[i - 1];
#pragma unroll UF
                            for (int j = i - 2; j >= 0; --j) {
                                dz[j] = fmadd(sd, st[j], dz[j]);
                                g[j + 1] = fmadd(sd, T(kInvFact[i - j - 1]), g[j + 1]);
                                sd *= z[j];
                            }
                        }
                    }
#pragma unroll UF
                    for (int i = 0; i < KMAX; ++i) {
                        if (i < k) {
                            if (use_lds) {
                                lds_add_shared(&mine[(s - s_lo) * slab + let[i]], dz[i]);
                            } else {
                                dev_add(&gx[s * d + let[i]], dz[i]);
                                dev_add(&gx[(s - 1) * d + let[i]], -dz[i]);
                            }
                        }
                    }
                }
            }
            if (use_lds) {
                __syncthreads();
                // point p = s_lo - 1 + q receives the sums of step p (chunk row q - 1) minus those of step p + 1 (row q)
                const int64_t n = s_hi - s_lo + 1;
                for (int64_t e = threadIdx.x; e < (n + 1) * d; e += blockDim.x) {
                    const int64_t q = e / d, j = e - q * d;
                    T sum = T(0);
                    for (int cpy = 0; cpy < copies; ++cpy) {
                        if (q >= 1) sum += acc[(q - 1) * slab + int64_t(cpy) * d + j];
                        if (q < n) sum -= acc[q * slab + int64_t(cpy) * d + j];
                    }
                    dev_add(&gx[(s_lo - 1 + q) * d + j], sum);
                }
                __syncthreads();
                for (int64_t j = threadIdx.x; j < n * slab; j += blockDim.x) acc[j] = T(0);
                if (s_hi - chunk >= 1) stage(s_hi - chunk);
                __syncthreads();
            }
        }
    }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct HostWords {
    std::vector<uint64_t> table;     // [start | out_start | degree], count entries each
    uint64_t count = 0, row = 0, max_degree = 0, letters = 0;
};

// copies the word list to the host, validates it and lays out the per-word offsets
static HostWords read_words(const uint64_t* multi_idx, uint64_t num_words, const uint64_t* degrees, uint64_t dimension,
                            bool prefix_layout, const char* who)
{
    HostWords h;
    h.count = num_words;
    if (num_words == 0) return h;
    if (!degrees) throw std::invalid_argument(std::string(who) + ": degrees is null");
    std::vector<uint64_t> deg(num_words);
    SIG_HIP(hipMemcpy(deg.data(), degrees, num_words * sizeof(uint64_t), hipMemcpyDeviceToHost));
    h.table.resize(3 * num_words);
    for (uint64_t w = 0; w < num_words; ++w) {
        h.table[w] = h.letters;
        h.table[num_words + w] = h.row;
        h.table[2 * num_words + w] = deg[w];
        h.letters = checked_mul(1, h.letters + deg[w], who);
        h.row += prefix_layout ? (deg[w] ? deg[w] : 1) : 1;
        h.max_degree = std::max(h.max_degree, deg[w]);
    }
    if (h.letters) {
        if (!multi_idx) throw std::invalid_argument(std::string(who) + ": multi_idx is null");
        std::vector<uint64_t> let(h.letters);
        SIG_HIP(hipMemcpy(let.data(), multi_idx, h.letters * sizeof(uint64_t), hipMemcpyDeviceToHost));
        for (uint64_t v : let)
            if (v >= dimension) throw std::invalid_argument(std::string(who) + ": multi_idx element out of range");
    }
    if (h.max_degree > uint64_t(kCoefMaxDegree))
        throw std::runtime_error(std::string(who) + ": words longer than 64 letters are not implemented in this build");
    return h;
}

template <typename F>
static void with_degree_bucket(uint64_t max_degree, F&& f)
{
    // (largest word length served, unroll factor)
    if (max_degree <= 4) f(IntC<4>{}, IntC<5>{});
    else if (max_degree <= 8) f(IntC<8>{}, IntC<9>{});
    else if (max_degree <= 16) f(IntC<16>{}, IntC<17>{});
    else f(IntC<kCoefMaxDegree>{}, IntC<1>{});
}

static WordList upload_words(const HostWords& h, const uint64_t* multi_idx, hipStream_t stream)
{
    uint64_t* dev = static_cast<uint64_t*>(workspace(6, h.table.size() * sizeof(uint64_t)));
    SIG_HIP(hipMemcpyAsync(dev, h.table.data(), h.table.size() * sizeof(uint64_t), hipMemcpyHostToDevice, stream));
    SIG_HIP(hipStreamSynchronize(stream));       // the host vector may go away once the caller returns
    return WordList{multi_idx, dev, dev + h.count, dev + 2 * h.count, h.count};
}

template <typename T>
static void sig_coef_impl(const T* path, T* out, const uint64_t* multi_idx, uint64_t num_words, const uint64_t* degrees,
                          uint64_t batch, uint64_t dimension, uint64_t length, bool prefixes)
{
    if (dimension == 0) throw std::invalid_argument("sig_coef received path of dimension 0");
    if (dimension > 0x3fffffff || length > (uint64_t(1) << 40)) throw std::invalid_argument("sig_coef_cuda: shape out of range");
    SIG_HIP(hipDeviceSynchronize());
    const HostWords h = read_words(multi_idx, num_words, degrees, dimension, true, "sig_coef");
    if (batch == 0 || num_words == 0) return;
    const uint64_t row = prefixes ? h.row : num_words;
    checked_mul(checked_mul(batch, row, "coefficients"), sizeof(T), "coefficients");
    checked_mul(checked_mul(checked_mul(batch, length, "path"), dimension, "path"), sizeof(T), "path");
    const uint64_t items = checked_mul(batch, num_words, "work items");
    hipStream_t stream = nullptr;
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    const WordList words = upload_words(h, multi_idx, stream);
    // points staged through LDS (a block per path and 256 words) when a chunk of at least 8 points fits 16 KB
    const uint64_t fit = uint64_t(16384) / (dimension * sizeof(T));
    const int chunk = int(std::min<uint64_t>(128, fit));
    with_degree_bucket(h.max_degree, [&](auto kc, auto uc) {
        constexpr int KMAX = decltype(kc)::value, UF = decltype(uc)::value;
        if (chunk >= 8) {
            const unsigned threads = num_words <= 64 ? 64u : unsigned(kBlock);
            const uint64_t gx = (num_words + threads - 1) / threads;
            if (gx > 0x7fffffffull) throw std::runtime_error("sig_coef_cuda: too many words");
            const dim3 grid{unsigned(gx), unsigned(std::min<uint64_t>(batch, 65535)), 1};
            hipLaunchKernelGGL((sig_coef_staged_kernel<T, KMAX, UF>), grid, dim3(threads),
                               size_t(chunk) * size_t(dimension) * sizeof(T), stream, path, out, words, int64_t(batch),
                               int64_t(dimension), int64_t(length), int64_t(row), int(prefixes), chunk);
        } else {
            hipLaunchKernelGGL((sig_coef_kernel<T, KMAX, UF>), dim3(grid_for(items)), dim3(kBlock), 0, stream, path, out, words,
                               int64_t(batch), int64_t(dimension), int64_t(length), int64_t(row), int(prefixes));
        }
    });
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void sig_coef_backprop_impl(const T* path, T* out, const T* coefs, const T* derivs, const uint64_t* multi_idx,
                                   uint64_t num_words, const uint64_t* degrees, uint64_t batch, uint64_t dimension,
                                   uint64_t length)
{
    if (dimension == 0) throw std::invalid_argument("sig_coef_backprop received path of dimension 0");
    if (dimension > 0x3fffffff || length > (uint64_t(1) << 40)) throw std::invalid_argument("sig_coef_backprop_cuda: shape out of range");
    SIG_HIP(hipDeviceSynchronize());
    const HostWords h = read_words(multi_idx, num_words, degrees, dimension, true, "sig_coef_backprop");
    const uint64_t path_elems = checked_mul(checked_mul(batch, length, "path"), dimension, "path");
    checked_mul(path_elems, sizeof(T), "path");
    if (path_elems == 0) return;
    hipStream_t stream = nullptr;
    hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(path_elems)), dim3(kBlock), 0, stream, out, int64_t(path_elems));
    if (num_words > 0 && length >= 2 && h.max_degree > 0) {
        const uint64_t items = checked_mul(batch, num_words, "work items");
        std::lock_guard<std::mutex> lk(g_ws_mutex);
        const WordList words = upload_words(h, multi_idx, stream);
        (void)items;
        // one block = up to 256 words of one path; per-channel sums in LDS unless the path is too wide for it
        const unsigned threads = num_words <= 64 ? 64u : unsigned(kBlock);
        const uint64_t gx = (num_words + threads - 1) / threads;
        if (gx > 0x7fffffffull) throw std::runtime_error("sig_coef_backprop_cuda: too many words");
        const int use_lds = dimension <= 4096 && 3 * dimension * sizeof(T) <= 65536;      // one step's sums + two points fit
        // LDS: `chunk` steps of `copies` private sets of per-channel sums, 32 KB at most, and the chunk's points
        int copies = use_lds ? int(std::max<uint64_t>(1, std::min<uint64_t>(8, 4096 / dimension))) : 1;
        auto steps_for = [&](int cp) { return uint64_t(32768) / (uint64_t(cp) * dimension * sizeof(T)); };
        while (copies > 1 && steps_for(copies) < 16) copies /= 2;
        int chunk = use_lds ? int(std::max<uint64_t>(1, std::min<uint64_t>(64, steps_for(copies)))) : 1;
        auto lds_for = [&](int ch) { return (size_t(ch) * size_t(copies) + size_t(ch) + 1) * size_t(dimension) * sizeof(T); };
        while (chunk > 1 && lds_for(chunk) > 65536) --chunk;       // sums and points together within 64 KB
        const size_t lds = use_lds ? lds_for(chunk) : 0;
        const dim3 grid{unsigned(gx), unsigned(std::min<uint64_t>(batch, 65535)), 1};
        with_degree_bucket(h.max_degree, [&](auto kc, auto uc) {
            constexpr int KMAX = decltype(kc)::value, UF = decltype(uc)::value;
            hipLaunchKernelGGL((sig_coef_bwd_kernel<T, KMAX, UF>), grid, dim3(threads), lds, stream, path, out, coefs, derivs,
                               words, int64_t(batch), int64_t(dimension), int64_t(length), int64_t(h.row), use_lds, copies,
                               chunk);
        });
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

}  // namespace sigamd

using namespace sigamd;

extern "C" {

CUSIG_AMD_API int sig_coef_cuda_f(const float* path, float* out, const uint64_t* multi_idx, uint64_t num_multi_idx,
                                  const uint64_t* degrees, uint64_t batch_size, uint64_t dimension, uint64_t length,
                                  bool prefixes) noexcept
{
    return guarded([&] { sig_coef_impl<float>(path, out, multi_idx, num_multi_idx, degrees, batch_size, dimension, length, prefixes); });
}
CUSIG_AMD_API int sig_coef_cuda_d(const double* path, double* out, const uint64_t* multi_idx, uint64_t num_multi_idx,
                                  const uint64_t* degrees, uint64_t batch_size, uint64_t dimension, uint64_t length,
                                  bool prefixes) noexcept
{
    return guarded([&] { sig_coef_impl<double>(path, out, multi_idx, num_multi_idx, degrees, batch_size, dimension, length, prefixes); });
}
CUSIG_AMD_API int sig_coef_backprop_cuda_f(const float* path, float* out, const float* coefs, const float* derivs,
                                           const uint64_t* multi_idx, uint64_t num_multi_idx, const uint64_t* degrees,
                                           uint64_t batch_size, uint64_t dimension, uint64_t length) noexcept
{
    return guarded([&] {
        sig_coef_backprop_impl<float>(path, out, coefs, derivs, multi_idx, num_multi_idx, degrees, batch_size, dimension, length);
    });
}
CUSIG_AMD_API int sig_coef_backprop_cuda_d(const double* path, double* out, const double* coefs, const double* derivs,
                                           const uint64_t* multi_idx, uint64_t num_multi_idx, const uint64_t* degrees,
                                           uint64_t batch_size, uint64_t dimension, uint64_t length) noexcept
{
    return guarded([&] {
        sig_coef_backprop_impl<double>(path, out, coefs, derivs, multi_idx, num_multi_idx, degrees, batch_size, dimension, length);
    });
}

}  // extern "C"
