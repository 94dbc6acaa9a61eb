// Expanded (tensor) logarithm of a signature and its backward pass, behind the reference's entry points
//   sig_to_log_sig_cuda_{f,d}, sig_to_log_sig_backprop_cuda_{f,d} with method 0
//   (decl siglib/cusig/cusig.h:391-431; arithmetic of siglib/cpsig/cp_tensor_log.h:40-113 forward, :164-221 backward).
// Methods 1 and 2 (Lyndon coordinates) need the reference's prepared Lyndon tables and are not part of this build.
//
// With x = sig - 1:   log(1 + x) = P_1,   P_k = x / k - x (x) P_{k+1},   P_{N+1} = 0,
// where P_k only needs levels <= N - k + 1.  One launch per k, one thread per coefficient.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>

#include "../../include/cusig_amd.h"
#include "sig_chen_adjoint.h"
#include "sig_host.h"
#include "sig_kernels.h"

namespace sigamd {

// P_out[r] = inv_k * x[r] - sum_{l=1..t-1} x_l[w_1..w_l] * P_in_{t-l}[w_{l+1}..w_t]   for the `count` coefficients of
// levels <= top.  x and the P buffers share one row layout (stride, off); `final` also clears the scalar slot.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void tensor_log_step_kernel(
    const T* __restrict__ X, const T* __restrict__ Pin, T* __restrict__ Pout, int64_t batch, DivBy<I> dv, I count,
    T inv_k, int64_t stride, int off, int64_t out_stride, int final)
{
    const I d = I(dv.d);
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = X + b * stride + off;
        const T* pin = Pin + b * stride + off;
        T* po = Pout + b * out_stride + off;
        for (I r = I(blockIdx.x) * kBlock + threadIdx.x; r < count; r += I(gridDim.x) * kBlock) {
            const WordPos<I> p = word_pos<I>(r, d);
            T acc = T(0);
            I pre = p.w, suf = 0, pw = 1;
            I a_lo = p.lo, a_sz = p.size;
            I b_lo = 0;
            for (int l = p.t - 1; l >= 1; --l) {        // split after l letters, as in the Chen product kernel
                const I q = dv.quot(pre);
                suf += (pre - q * d) * pw;
                pw *= d;
                pre = q;
                a_sz = dv.quot(a_sz);
                a_lo -= a_sz;
                acc = fmadd(x[a_lo + pre], pin[b_lo + suf], acc);
                b_lo += pw;
            }
            po[r] = inv_k * x[r] - acc;
            if (final && off && r == 0) po[-off] = T(0);
        }
    }
}

// after the adjoint of x (x) P_{k+1} (tmpA w.r.t. x, tmpB w.r.t. P_{k+1}):
//   g_next = -tmpB,   dx += -tmpA + g_next / (k + 1)      over the `count` coefficients of levels <= N - k + 1
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void tensor_log_bwd_update_kernel(
    T* __restrict__ dx, T* __restrict__ g_next, const T* __restrict__ tmpA, const T* __restrict__ tmpB, int64_t batch,
    I count, I count_next, T inv_next, int64_t stride, int off)
{
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const int64_t base = b * stride + off;
        for (I r = I(blockIdx.x) * kBlock + threadIdx.x; r < count; r += I(gridDim.x) * kBlock) {
            T v = dx[base + r] - tmpA[base + r];
            if (r < count_next) {
                const T gn = -tmpB[base + r];
                g_next[base + r] = gn;
                v = fmadd(gn, inv_next, v);
            }
            dx[base + r] = v;
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
    if (method != 0)
        throw std::runtime_error(std::string(who) + ": methods 1 and 2 (Lyndon coordinates) are not implemented in this "
                                 "build; use method 0 (expanded tensor logarithm)");
}

// number of coefficients of levels 1 .. t
static uint64_t coef_count(uint64_t d, uint64_t t) { return sig_length_u64(d, t) - 1; }

// runs the recursion; P_k (k >= 2) lands in p_of(k), P_1 in `out`
template <typename T, typename PofK>
static void run_tensor_log(const T* sig, T* out, uint64_t batch, uint64_t dimension, uint64_t degree, const SigShape& s,
                           hipStream_t stream, PofK&& p_of)
{
    launch_indexed(s.n_coef, 1, batch, [&](auto ix, dim3) {
        using I = decltype(ix);
        const DivBy<I> dv(dimension);
        for (uint64_t k = degree; k >= 1; --k) {
            const uint64_t count = coef_count(dimension, degree - k + 1);
            const T* pin = k == degree ? sig : p_of(k + 1);       // unused when k == degree: only level 1 is computed
            T* pout = k == 1 ? out : p_of(k);
            launch_indexed(0, count, batch, [&](auto, dim3 grid) {
                hipLaunchKernelGGL((tensor_log_step_kernel<T, I>), grid, dim3(kBlock), 0, stream, sig, pin, pout, int64_t(batch),
                                   dv, I(count), T(1) / T(k), int64_t(s.stride), s.off, int64_t(s.stride), int(k == 1));
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
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term) hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch));
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    T* ws = degree >= 2 ? static_cast<T*>(workspace(7, checked_mul(bytes, 2, "workspace"))) : nullptr;
    const uint64_t elems = batch * s.stride;
    run_tensor_log<T>(sig, out, batch, dimension, degree, s, stream, [&](uint64_t k) { return ws + (k & 1) * elems; });
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
    hipStream_t stream = nullptr;
    if (s.n_coef == 0) {
        if (scalar_term) hipLaunchKernelGGL((zero_kernel<T>), dim3(grid_for(batch)), dim3(kBlock), 0, stream, out, int64_t(batch));
        SIG_HIP(hipGetLastError());
        SIG_HIP(hipStreamSynchronize(stream));
        return;
    }
    std::lock_guard<std::mutex> lk(g_ws_mutex);
    const uint64_t elems = batch * s.stride;
    // P_1 (discarded), P_2 .. P_N, two adjoint buffers, two product-adjoint buffers
    T* ws = degree >= 2 ? static_cast<T*>(workspace(7, checked_mul(bytes, degree + 4, "workspace"))) : nullptr;
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
        run_tensor_log<T>(sig, p_base, batch, dimension, degree, s, stream, [&](uint64_t k) { return p_base + (k - 1) * elems; });
        const T* g = derivs;
        for (uint64_t k = 1; k < degree; ++k) {
            const uint64_t top = degree - k + 1;          // levels of g_k
            const SigShape sk{coef_count(dimension, top), s.stride, s.off};
            launch_combine_bwd<T>(g, tmpA, tmpB, sig, p_base + k * elems, batch, dimension, top, sk, stream, /*identity=*/0);
            T* g_next = g_buf[k & 1];
            const uint64_t count = sk.n_coef, count_next = coef_count(dimension, top - 1);
            launch_indexed(s.n_coef, count, batch, [&](auto ix, dim3 grid) {
                using I = decltype(ix);
                hipLaunchKernelGGL((tensor_log_bwd_update_kernel<T, I>), grid, dim3(kBlock), 0, stream, out, g_next,
                                   (const T*)tmpA, (const T*)tmpB, int64_t(batch), I(count), I(count_next), T(1) / T(k + 1),
                                   int64_t(s.stride), s.off);
            });
            g = g_next;
        }
    }
    SIG_HIP(hipGetLastError());
    SIG_HIP(hipStreamSynchronize(stream));
}

}  // namespace sigamd

using namespace sigamd;

extern "C" {

CUSIG_AMD_API int sig_to_log_sig_cuda_f(const float* sig, float* out, uint64_t batch_size, uint64_t dimension, uint64_t degree,
                                        int method, bool scalar_term) noexcept
{
    return guarded([&] { sig_to_log_sig_impl<float>(sig, out, batch_size, dimension, degree, method, scalar_term); });
}
CUSIG_AMD_API int sig_to_log_sig_cuda_d(const double* sig, double* out, uint64_t batch_size, uint64_t dimension,
                                        uint64_t degree, int method, bool scalar_term) noexcept
{
    return guarded([&] { sig_to_log_sig_impl<double>(sig, out, batch_size, dimension, degree, method, scalar_term); });
}
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_f(const float* sig, float* out, const float* log_sig_derivs, uint64_t batch_size,
                                                 uint64_t dimension, uint64_t degree, int method, bool scalar_term) noexcept
{
    return guarded([&] {
        sig_to_log_sig_backprop_impl<float>(sig, out, log_sig_derivs, batch_size, dimension, degree, method, scalar_term);
    });
}
CUSIG_AMD_API int sig_to_log_sig_backprop_cuda_d(const double* sig, double* out, const double* log_sig_derivs,
                                                 uint64_t batch_size, uint64_t dimension, uint64_t degree, int method,
                                                 bool scalar_term) noexcept
{
    return guarded([&] {
        sig_to_log_sig_backprop_impl<double>(sig, out, log_sig_derivs, batch_size, dimension, degree, method, scalar_term);
    });
}

}  // extern "C"
