// Logarithm of a signature and its backward pass, behind the reference's entry points
//   sig_to_log_sig_cuda_{f,d}, sig_to_log_sig_backprop_cuda_{f,d}, prepare_log_sig_cuda, clear_cache_cuda
//   (decl siglib/cusig/cusig.h:391-447, 616-626; arithmetic of siglib/cpsig/cp_tensor_log.h:40-113 forward,
//   :140-170 Lyndon coordinates, :164-221 backward).
// Method 0: expanded (tensor) logarithm.  Methods 1 and 2: its coordinates at the Lyndon words resp. in the Lyndon
// basis, from tables prepared on the host per (device, dimension, degree) (sig_lyndon.h); as in the reference they
// must have been prepared with prepare_log_sig_cuda (status 5 otherwise).  Method 3 (BCH) is not part of this build.
//
// With x = sig - 1:   log(1 + x) = P_1,   P_k = x / k - x (x) P_{k+1},   P_{N+1} = 0,
// where P_k only needs levels <= N - k + 1.  One launch per k, one thread per coefficient.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <string>
#include <tuple>
#include <vector>

#include "../../include/cusig_amd.h"
#include "sig_chen_adjoint.h"
#include "sig_host.h"
#include "sig_kernels.h"
#include "sig_lyndon.h"

namespace sigamd {

// P_out[r] = inv_k * x[r] - sum_{l=1..t-1} x_l[w_1..w_l] * P_in_{t-l}[w_{l+1}..w_t]   for the `count` coefficients of
// levels <= top.  x and the P buffers share one row layout (stride, off); `final` also clears the scalar slot.
template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void tensor_log_step_kernel(
    const T* __restrict__ X, const T* __restrict__ Pin, T* __restrict__ Pout, int64_t batch, DivBy<I> dv,
    I items /* chen_items(d, levels, FAN) */, T inv_k, int64_t stride, int off, int64_t out_stride, int final,
    I low_n /* chen_low_count: dynamic LDS of 2 * low_n entries; 0 = none */)
{
    extern __shared__ double log_low_raw[];
    T* xl = reinterpret_cast<T*>(log_low_raw);
    T* pl = xl + low_n;
    for (int64_t b = xcd_block_2d().y; b < batch; b += gridDim.y) {
        const T* x = X + b * stride + off;
        const T* pin = Pin + b * stride + off;
        T* po = Pout + b * out_stride + off;
        if (low_n) stage_low_levels(xl, pl, x, pin, low_n);
        for (I it = I(xcd_block_2d().x) * kBlock + threadIdx.x; it < items; it += I(gridDim.x) * kBlock) {
            // the splits after l = 1 .. t-1 letters, several first letters per thread as in the Chen product kernels
            if (low_n) chen_fan<T, I, FAN, true>(x, pin, it, dv, [&](I r, T sum) { po[r] = inv_k * x[r] - sum; }, xl, pl, low_n);
            else chen_fan<T, I, FAN>(x, pin, it, dv, [&](I r, T sum) { po[r] = inv_k * x[r] - sum; });
            if (final && off && it == 0) po[-off] = T(0);
        }
    }
}

// The same step evaluated only at the `count` coefficients listed in `index` (positions in a scalar-free row): the last
// step of the recursion when only the Lyndon words' coordinates of the logarithm are wanted (a fifth of the row at
// d = 10, degree 5).  With one output per work item the item number of the Chen product kernels IS the coefficient's
// position, so the listed positions are fed to chen_fan directly.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void tensor_log_step_at_kernel(
    const T* __restrict__ X, const T* __restrict__ Pin, T* __restrict__ Pout, int64_t batch, DivBy<I> dv,
    const uint64_t* __restrict__ index, int64_t count, T inv_k, int64_t stride, int off, int64_t out_stride)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = X + b * stride + off;
        const T* pin = Pin + b * stride + off;
        T* po = Pout + b * out_stride + off;
        for (int64_t i = int64_t(blockIdx.x) * kBlock + threadIdx.x; i < count; i += int64_t(gridDim.x) * kBlock)
            chen_fan<T, I, 1>(x, pin, I(index[i]), dv, [&](I r, T sum) { po[r] = inv_k * x[r] - sum; });
    }
}

// after the adjoint of x (x) P_{k+1} with -P_{k+1} as the left factor's partner (tmpB w.r.t. P_{k+1}; w.r.t. x:
// -tmpA, which the k = 1 call has already added to g inside dx and the later calls leave in `neg_a`):
//   g_next = -tmpB,   dx += neg_a + g_next / (k + 1)      over the `count_next` coefficients of levels <= N - k
// (neither gradient has a term at level N - k + 1: the Chen product's adjoint without its dC term stops one level short)
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void tensor_log_bwd_update_kernel(
    T* __restrict__ dx, T* __restrict__ g_next, const T* __restrict__ neg_a, const T* __restrict__ tmpB, int64_t batch,
    I count_next, T inv_next, int64_t stride, int off)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const int64_t base = b * stride + off;
        for (I r = I(blockIdx.x) * kBlock + threadIdx.x; r < count_next; r += I(gridDim.x) * kBlock) {
            const T gn = -tmpB[base + r];
            g_next[base + r] = gn;
            T v = dx[base + r];
            if (neg_a) v += neg_a[base + r];
            dx[base + r] = fmadd(gn, inv_next, v);
        }
    }
}

// dx = g (the k = 1 term of the adjoint), scalar slot zero
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void tensor_log_bwd_init_kernel(
    T* __restrict__ dx, const T* __restrict__ g, int64_t batch, I count, int64_t stride, int off)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const int64_t base = b * stride + off;
        for (I r = I(blockIdx.x) * kBlock + threadIdx.x; r < count; r += I(gridDim.x) * kBlock) {
            dx[base + r] = g[base + r];
            if (off && r == 0) dx[b * stride] = T(0);
        }
    }
}

static void check_method(int method, const char* who)
{
    if (method < 0 || method > 2) throw std::invalid_argument(std::string(who) + ": method must be 0, 1 or 2");
}

// ---------------------------------------------------------------------------
// Lyndon coordinates: prepared tables on the device
// ---------------------------------------------------------------------------
struct CacheMissing : CodedError {
    explicit CacheMissing(const char* what_) : CodedError(5, what_) {}
};

struct DeviceLyndon {
    int method = 0;
    uint64_t count = 0;                                  // Lyndon words
    uint64_t* index = nullptr;                           // their positions in a scalar-free row
    uint64_t *row_ptr = nullptr, *t_row_ptr = nullptr;   // strictly lower part of M^-1 and of its transpose (CSR)
    uint32_t *col = nullptr, *t_col = nullptr;
    uint64_t* col_pos = nullptr;                         // index[col[k]]: the row position the k-th entry of M^-1 reads
    int32_t *val = nullptr, *t_val = nullptr;
    void release() noexcept
    {
        for (void* p : {(void*)index, (void*)row_ptr, (void*)t_row_ptr, (void*)col, (void*)t_col, (void*)val, (void*)t_val,
                        (void*)col_pos})
            if (p) (void)hipFree(p);
        *this = DeviceLyndon();
    }
};
static std::mutex g_lyndon_mutex;
static std::map<std::tuple<int, uint64_t, uint64_t>, DeviceLyndon> g_lyndon;       // (device, dimension, degree)

template <typename V>
static V* upload(const std::vector<V>& host)
{
    V* dev = nullptr;
    SIG_HIP(hipMalloc(reinterpret_cast<void**>(&dev), std::max<size_t>(host.size(), 1) * sizeof(V)));
    if (!host.empty()) SIG_HIP(hipMemcpy(dev, host.data(), host.size() * sizeof(V), hipMemcpyHostToDevice));
    return dev;
}

static void prepare_lyndon(uint64_t dimension, uint64_t degree, int method)
{
    if (method == 0) return;
    if (method == 3) throw std::runtime_error("prepare_log_sig_cuda: method 3 (BCH) is not implemented in this build");
    if (method < 0 || method > 3) throw std::invalid_argument("log signature method must be 1, 2, or 3");
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    // order of the two locks everywhere: workspace mutex first (held by every call that may be using a table)
    std::lock_guard<std::mutex> ws_lk(g_ws_mutex);
    std::lock_guard<std::mutex> lk(g_lyndon_mutex);
    DeviceLyndon& slot = g_lyndon[std::make_tuple(dev, dimension, degree)];
    if (slot.method >= method) return;                   // preparing for method 2 also serves method 1
    const LyndonTables t = build_lyndon_tables(dimension, degree, method);
    DeviceLyndon fresh;
    try {
        fresh.method = method;
        fresh.count = t.index.size();
        fresh.index = upload(t.index);
        if (method == 2) {
            fresh.row_ptr = upload(t.row_ptr);
            fresh.t_row_ptr = upload(t.t_row_ptr);
            fresh.col = upload(t.col);
            fresh.t_col = upload(t.t_col);
            std::vector<uint64_t> pos(t.col.size());
            for (size_t k = 0; k < pos.size(); ++k) pos[k] = t.index[t.col[k]];
            fresh.col_pos = upload(pos);
            fresh.val = upload(t.val);
            fresh.t_val = upload(t.t_val);
        }
    } catch (...) {
        fresh.release();
        throw;
    }
    slot.release();
    slot = fresh;
}

void clear_lyndon_tables() noexcept
{
    std::lock_guard<std::mutex> ws_lk(g_ws_mutex);      // no call is using a table while they are freed
    std::lock_guard<std::mutex> lk(g_lyndon_mutex);
    int cur = 0;
    const bool have = hipGetDevice(&cur) == hipSuccess;
    for (auto& kv : g_lyndon) {
        if (have && hipSetDevice(std::get<0>(kv.first)) == hipSuccess) kv.second.release();
    }
    if (have) (void)hipSetDevice(cur);
    g_lyndon.clear();
    (void)hipGetLastError();
}

static DeviceLyndon find_lyndon(uint64_t dimension, uint64_t degree, int method)
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lk(g_lyndon_mutex);
    auto it = g_lyndon.find(std::make_tuple(dev, dimension, degree));
    if (it == g_lyndon.end() || it->second.method < method) throw CacheMissing("Could not find prepared cache");
    return it->second;
}

// out[b][i] = x[b][index[i]] (method 1) plus sum_k val[k] * x[b][col_pos[k]] over the row's entries (method 2;
// col_pos[k] = index[col[k]], resolved when the tables are prepared)
template <typename T>
__global__ __launch_bounds__(kBlock) void lyndon_compress_kernel(
    const T* __restrict__ expanded, T* __restrict__ out, int64_t batch, int64_t count, int64_t stride, int off,
    const uint64_t* __restrict__ index, const uint64_t* __restrict__ row_ptr, const uint64_t* __restrict__ col_pos,
    const int32_t* __restrict__ val)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = expanded + b * stride + off;
        for (int64_t i = int64_t(blockIdx.x) * kBlock + threadIdx.x; i < count; i += int64_t(gridDim.x) * kBlock) {
            T acc = x[index[i]];
            if (row_ptr)
                for (uint64_t k = row_ptr[i]; k < row_ptr[i + 1]; ++k) acc = fmadd(T(val[k]), x[col_pos[k]], acc);
            out[b * count + i] = acc;
        }
    }
}

// the transpose: dx[b][index[j]] = g[b][j] + sum_k t_val[k] * g[b][t_col[k]]; every other entry of dx must be zero
// beforehand
template <typename T>
__global__ __launch_bounds__(kBlock) void lyndon_expand_kernel(
    const T* __restrict__ g, T* __restrict__ dx, int64_t batch, int64_t count, int64_t stride, int off,
    const uint64_t* __restrict__ index, const uint64_t* __restrict__ t_row_ptr, const uint32_t* __restrict__ t_col,
    const int32_t* __restrict__ t_val)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* gb = g + b * count;
        for (int64_t j = int64_t(blockIdx.x) * kBlock + threadIdx.x; j < count; j += int64_t(gridDim.x) * kBlock) {
            T acc = gb[j];
            if (t_row_ptr)
                for (uint64_t k = t_row_ptr[j]; k < t_row_ptr[j + 1]; ++k) acc = fmadd(T(t_val[k]), gb[t_col[k]], acc);
            dx[b * stride + off + index[j]] = acc;
        }
    }
}

// number of coefficients of levels 1 .. t
static uint64_t coef_count(uint64_t d, uint64_t t) { return sig_length_u64(d, t) - 1; }

// runs the recursion down to k = k_min; P_k (k >= 2) lands in p_of(k), P_1 in `out`.  sign = -1 computes -P_k instead
// (the recursion is linear in x / k, the only place the sign enters)
template <typename T, typename PofK>
static void run_tensor_log(const T* sig, T* out, uint64_t batch, uint64_t dimension, uint64_t degree, const SigShape& s,
                           hipStream_t stream, PofK&& p_of, uint64_t k_min = 1, int sign = 1)
{
    launch_indexed(s.n_coef, 1, batch, [&](auto ix, dim3) {
        using I = decltype(ix);
        const DivBy<I> dv(dimension);
        for (uint64_t k = degree; k >= k_min; --k) {
            const uint64_t count = coef_count(dimension, degree - k + 1);
            const T* pin = k == degree ? sig : p_of(k + 1);       // unused when k == degree: only level 1 is computed
            T* pout = k == 1 ? out : p_of(k);
            with_chen_fan(dimension, [&](auto fan) {
                constexpr int FAN = decltype(fan)::value;
                const uint64_t items = chen_items(dimension, degree - k + 1, FAN);
                // the short levels of x and P_{k+1} in LDS (the step with one level computes no product and needs none)
                const uint64_t blocks = (items + kBlock - 1) / kBlock * batch;
                const uint64_t low_n = degree - k + 1 >= 3 ? chen_low_count(dimension, degree - k + 1, sizeof(T), blocks) : 0;
                const uint64_t per_thread = low_n ? chen_low_items_per_thread(low_n, blocks) : 1;
                launch_indexed(0, (items + per_thread - 1) / per_thread, batch, [&](auto, dim3 grid) {
                    hipLaunchKernelGGL((tensor_log_step_kernel<T, I, FAN>), grid, dim3(kBlock), 2 * low_n * sizeof(T), stream, sig,
                                       pin, pout, int64_t(batch), dv, I(items), T(sign) / T(k), int64_t(s.stride), s.off,
                                       int64_t(s.stride), int(k == 1), I(low_n));
                });
            });
        }
    });
}

template <typename T>
static void sig_to_log_sig_impl(const T* sig, T* out, uint64_t batch, uint64_t dimension, uint64_t degree, int method,
                                bool scalar_term)
{
    check_method(method, "sig_to_log_sig_cuda");
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_to_log_sig_cuda");
    if (batch == 0) return;
    const uint64_t bytes = checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    // The prepared tables are looked up and used under the workspace mutex, which prepare / clear / shutdown also take
    // before they free a table: a table found here stays alive until this call's kernels have finished.
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    const DeviceLyndon lyn = method ? find_lyndon(dimension, degree, method) : DeviceLyndon();
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        // degree 0: the compressed forms are empty, the expanded one holds the scalar slot
        if (scalar_term && !method) hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch));
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    T* ws = degree >= 2 ? static_cast<T*>(workspace(7, checked_mul(bytes, 2, "workspace"))) : nullptr;
    const uint64_t elems = batch * s.stride;
    // Lyndon coordinates are read off the expanded logarithm, which then lives in a scratch copy
    T* expanded = method ? static_cast<T*>(workspace(14, bytes)) : out;
    if (method && degree >= 2) {
        // only the Lyndon words' coordinates are read below: the last step, most of the work, is evaluated at those
        run_tensor_log<T>(sig, expanded, batch, dimension, degree, s, stream, [&](uint64_t k) { return ws + (k & 1) * elems; }, 2);
        launch_indexed(s.n_coef, lyn.count, batch, [&](auto ix, dim3 grid) {
            using I = decltype(ix);
            hipLaunchKernelGGL((tensor_log_step_at_kernel<T, I>), grid, dim3(kBlock), 0, stream, sig, (const T*)(ws + (2 & 1) * elems),
                               expanded, int64_t(batch), DivBy<I>(dimension), (const uint64_t*)lyn.index, int64_t(lyn.count), T(1),
                               int64_t(s.stride), s.off, int64_t(s.stride));
        });
    } else {
        run_tensor_log<T>(sig, expanded, batch, dimension, degree, s, stream, [&](uint64_t k) { return ws + (k & 1) * elems; });
    }
    if (method) {
        launch_indexed(0, lyn.count, batch, [&](auto, dim3 grid) {
            hipLaunchKernelGGL((lyndon_compress_kernel<T>), grid, dim3(kBlock), 0, stream, (const T*)expanded, out, int64_t(batch),
                               int64_t(lyn.count), int64_t(s.stride), s.off, (const uint64_t*)lyn.index,
                               (const uint64_t*)(method == 2 ? lyn.row_ptr : nullptr), (const uint64_t*)lyn.col_pos,
                               (const int32_t*)lyn.val);
        });
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

template <typename T>
static void sig_to_log_sig_backprop_impl(const T* sig, T* out, const T* derivs, uint64_t batch, uint64_t dimension,
                                         uint64_t degree, int method, bool scalar_term)
{
    check_method(method, "sig_to_log_sig_backprop_cuda");
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_to_log_sig_backprop_cuda");
    if (batch == 0) return;
    const uint64_t bytes = checked_mul(checked_mul(batch, s.stride, "signature"), sizeof(T), "signature");
    SIG_HIP(hipDeviceSynchronize());
    std::lock_guard<std::mutex> lk(g_ws_mutex);      // see sig_to_log_sig_impl
    const DeviceLyndon lyn = method ? find_lyndon(dimension, degree, method) : DeviceLyndon();
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term) hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch));
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    const uint64_t elems = batch * s.stride;
    if (method) {
        // gradient w.r.t. the expanded logarithm: the transposed coordinate map, zero off the Lyndon words
        T* dexp = static_cast<T*>(workspace(15, bytes));
        hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(elems)), dim3(kBlock), 0, stream, dexp, int64_t(elems));
        launch_indexed(0, lyn.count, batch, [&](auto, dim3 grid) {
            hipLaunchKernelGGL((lyndon_expand_kernel<T>), grid, dim3(kBlock), 0, stream, derivs, dexp, int64_t(batch),
                               int64_t(lyn.count), int64_t(s.stride), s.off, (const uint64_t*)lyn.index,
                               (const uint64_t*)(method == 2 ? lyn.t_row_ptr : nullptr), (const uint32_t*)lyn.t_col,
                               (const int32_t*)lyn.t_val);
        });
        derivs = dexp;
    }
    // -P_2 .. -P_N (the slot of P_1 stays unused), two adjoint buffers, two product-adjoint buffers
    T* ws = degree >= 2 ? static_cast<T*>(workspace(7, checked_mul(bytes, degree + 4, "workspace"))) : nullptr;
    if (degree < 2)
        launch_indexed(s.n_coef, s.n_coef, batch, [&](auto ix, dim3 grid) {
            using I = decltype(ix);
            hipLaunchKernelGGL((tensor_log_bwd_init_kernel<T, I>), grid, dim3(kBlock), 0, stream, out, derivs, int64_t(batch),
                               I(s.n_coef), int64_t(s.stride), s.off);
        });
    if (degree >= 2) {
        T* p_base = ws;                                   // P_k at p_base + (k - 1) * elems
        T* g_buf[2] = {ws + degree * elems, ws + (degree + 1) * elems};
        T* tmpA = ws + (degree + 2) * elems;
        T* tmpB = ws + (degree + 3) * elems;
        // the backward pass never reads P_1, and takes the others negated: the left factor's gradient of
        // x (x) (-P_{k+1}) is the term dx needs, sign included
        run_tensor_log<T>(sig, p_base, batch, dimension, degree, s, stream, [&](uint64_t k) { return p_base + (k - 1) * elems; },
                          2, -1);
        const T* g = derivs;
        for (uint64_t k = 1; k < degree; ++k) {
            const uint64_t top = degree - k + 1;          // levels of g_k
            const SigShape sk{coef_count(dimension, top), s.stride, s.off};
            // k = 1: the left factor's gradient keeps its dC term and lands in `out`, which is then g - tmpA already
            launch_combine_bwd<T>(g, k == 1 ? out : tmpA, tmpB, sig, p_base + k * elems, batch, dimension, top, sk, stream,
                                  /*identity=*/k == 1 ? 1 : 0);
            T* g_next = g_buf[k & 1];
            const uint64_t count_next = coef_count(dimension, top - 1);
            launch_indexed(s.n_coef, count_next, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                hipLaunchKernelGGL((tensor_log_bwd_update_kernel<T, I>), grid, dim3(kBlock), 0, stream, out, g_next,
                                   k == 1 ? static_cast<const T*>(nullptr) : (const T*)tmpA, (const T*)tmpB, int64_t(batch),
                                   I(count_next), T(1) / T(k + 1), int64_t(s.stride), s.off);
            });
            g = g_next;
        }
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

// values per path in the compressed (methods 1, 2) or expanded (method 0) logarithm
static uint64_t log_row_len(uint64_t dimension, uint64_t degree, int method, const SigShape& s)
{
    if (!method) return s.stride;
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    return find_lyndon(dimension, degree, method).count;
}

// the two operators with the batch taken in halves when the device cannot hold the workspace of the whole call
// (siglib/cusig/cu_runtime_utils.h:103-105,212-235)
template <typename T>
static void sig_to_log_sig_entry(const T* sig, T* out, uint64_t batch, uint64_t dimension, uint64_t degree, int method,
                                 bool scalar_term)
{
    check_method(method, "sig_to_log_sig_cuda");
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_to_log_sig_cuda");
    const uint64_t row = batch ? log_row_len(dimension, degree, method, s) : 0;
    split_on_bad_alloc(batch, "sig_to_log_sig", [&](uint64_t first, uint64_t count) {
        sig_to_log_sig_impl<T>(sig + first * s.stride, out + first * row, count, dimension, degree, method, scalar_term);
    });
}

template <typename T>
static void sig_to_log_sig_backprop_entry(const T* sig, T* out, const T* derivs, uint64_t batch, uint64_t dimension,
                                          uint64_t degree, int method, bool scalar_term)
{
    check_method(method, "sig_to_log_sig_backprop_cuda");
    const SigShape s = sig_shape(dimension, degree, scalar_term, "sig_to_log_sig_backprop_cuda");
    const uint64_t row = batch ? log_row_len(dimension, degree, method, s) : 0;
    split_on_bad_alloc(batch, "sig_to_log_sig_backprop", [&](uint64_t first, uint64_t count) {
        sig_to_log_sig_backprop_impl<T>(sig + first * s.stride, out + first * s.stride, derivs + first * row, count, dimension,
                                        degree, method, scalar_term);
    });
}

}  // namespace sigamd

using namespace sigamd;

extern "C" {

CUSIG_AMD_API int sig_to_log_sig_cuda_f(const float* sig, float* out, uint64_t batch_size, uint64_t dimension, uint64_t degree,
                                        int method, bool scalar_term) noexcept
{
    return guarded([&] { sig_to_log_sig_entry<float>(sig, out, batch_size, dimension, degree, method, scalar_term); });
}
CUSIG_AMD_API int sig_to_log_sig_cuda_d(const double* sig, double* out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t degree, int method, bool scalar_term) noexcept
{
    return guarded([&] { sig_to_log_sig_entry<double>(sig, out, batch_size, dimension, degree, method, scalar_term); });
}
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_f(const float* sig, float* out, const float* log_sig_derivs, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t degree, int method, bool scalar_term) noexcept
{
    return guarded([&] {
        sig_to_log_sig_backprop_entry<float>(sig, out, log_sig_derivs, batch_size, dimension, degree, method, scalar_term);
    });
}
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_d(const double* sig, double* out, const double* log_sig_derivs,
                                                 uint64_t batch_size, uint64_t dimension, uint64_t degree, int method,
                                                 bool scalar_term) noexcept
{
    return guarded([&] {
        sig_to_log_sig_backprop_entry<double>(sig, out, log_sig_derivs, batch_size, dimension, degree, method, scalar_term);
    });
}

/* Replaces prepare_log_sig_cuda (siglib/cusig/cusig.h:447): builds and uploads the Lyndon tables of (dimension, degree) for
 * the current device.  use_disk is accepted and ignored: tables are rebuilt in memory (milliseconds for the sizes
 * a signature of that shape allows). */
CUSIG_AMD_API int prepare_log_sig_cuda(uint64_t dimension, uint64_t degree, int method, bool) noexcept
{
    return guarded([&] { prepare_lyndon(dimension, degree, method); });
}

/* Host-only view of the tables prepare_log_sig_cuda uploads (needs no GPU): first call with null arrays for the sizes,
 * then with arrays of `count` indices, `count + 1` row offsets and `nnz` columns / values (strictly lower part of the
 * inverse projection; empty for method 1). */
CUSIG_AMD_API int cusig_amd_lyndon_tables(uint64_t dimension, uint64_t degree, int method, uint64_t* count, uint64_t* nnz,
                                          uint64_t* index, uint64_t* row_ptr, uint32_t* col, int32_t* val) noexcept
{
    return guarded([&] {
        if (method != 1 && method != 2) throw std::invalid_argument("cusig_amd_lyndon_tables: method must be 1 or 2");
        const LyndonTables t = build_lyndon_tables(dimension, degree, method);
        if (count) *count = t.index.size();
        if (nnz) *nnz = t.col.size();
        if (index) std::copy(t.index.begin(), t.index.end(), index);
        if (row_ptr) std::copy(t.row_ptr.begin(), t.row_ptr.end(), row_ptr);
        if (col) std::copy(t.col.begin(), t.col.end(), col);
        if (val) std::copy(t.val.begin(), t.val.end(), val);
    });
}

/* Replaces clear_cache_cuda (siglib/cusig/cusig.h:626): drops every prepared table on every device. */
CUSIG_AMD_API int clear_cache_cuda(bool) noexcept
{
    return guarded([&] { clear_lyndon_tables(); });
}

}  // extern "C"
