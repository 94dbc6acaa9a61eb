// Degree-3 backward for wide paths as two matrix products on the matrix cores plus one scan.
//
// With S' = S (x) exp(z) (siglib/cpsig/cp_signature.h:426-500 for the step, :909-1019 for its adjoint), degree 3:
//   S1' = S1 + z,   S2' = S2 + S1 (x) z + z (x) z / 2,   S3' = S3 + S2 (x) z + S1 (x) z (x) z / 2 + z (x) z (x) z / 6.
// The adjoint a3 of the level-3 state never changes: it is the upstream gradient G3 (d^2 x d as a matrix).  Every
// d^3-sized piece of the backward pass is therefore one of two products with that constant matrix:
//   Y_t = G3 z_t                       (d^2 values per step;  Y = Z G3^T over all steps: [L x d] [d x d^2])
//   W_t = G3^T V_t                     (d values per step;    W = V G3:                  [L x d^2] [d^2 x d])
// with V_t = S2 + S1 (x) z_t / 2 + z_t (x) z_t / 6 (S = state before step t).  Both run as strided-batched GEMMs in
// rocBLAS (plain library products; the library is opened at first use, and its absence only means that the sweep
// kernels serve these shapes).  Between them one scan kernel walks the steps backwards per coefficient (i, j): it
// recovers S2 by un-multiplying, carries a2 <- a2 + Y_t, overwrites Y_t with V_t in place, and adds the d^2-sized
// terms of the increment gradient (row and column sums of a2 and Y against S1 and z).  A last kernel adds the level-1
// adjoint, a running sum over the steps.
//
//   a2[i,j] = a2'[i,j] + Y[i,j]                       a1[i] = a1'[i] + sum_j (a2' + Y / 2)[i,j] z[j]
//   dz[m] = a1'[m] + W[m] + sum_i a2'[i,m] (S1[i] + z[i] / 2) + sum_i Y[i,m] (S1[i] / 2 + z[i] / 6)
//                         + sum_j a2'[m,j] z[j] / 2 + sum_j Y[m,j] z[j] / 6
#pragma once
#include <dlfcn.h>
#include <hip/hip_runtime.h>

#include <cstdint>
#include <map>
#include <stdexcept>

#include "sig_kernels.h"

namespace sigamd {

constexpr int kDeg3RowsPerThread = 8;       // coefficients (i, j) a thread carries: i in a group of 8, one j
constexpr int kDeg3MaxDim = 1024;

// ---- rocBLAS, opened at first use ----------------------------------------------------------------------------------
struct RocBlas {
    using Handle = void*;
    int (*create)(Handle*) = nullptr;
    int (*destroy)(Handle) = nullptr;
    int (*set_stream)(Handle, hipStream_t) = nullptr;
    int (*sgemm)(Handle, int, int, int, int, int, const float*, const float*, int, int64_t, const float*, int, int64_t,
                 const float*, float*, int, int64_t, int) = nullptr;
    int (*dgemm)(Handle, int, int, int, int, int, const double*, const double*, int, int64_t, const double*, int, int64_t,
                 const double*, double*, int, int64_t, int) = nullptr;
    bool tried = false, ok = false;
    std::map<int, Handle> handles;      // per device
};
static RocBlas g_rocblas;               // guarded by the workspace mutex

static bool rocblas_ready()
{
    RocBlas& r = g_rocblas;
    if (!r.tried) {
        r.tried = true;
        void* lib = dlopen("librocblas.so.5", RTLD_NOW | RTLD_LOCAL);
        if (!lib) lib = dlopen("librocblas.so", RTLD_NOW | RTLD_LOCAL);
        if (lib) {
            r.create = reinterpret_cast<decltype(r.create)>(dlsym(lib, "rocblas_create_handle"));
            r.destroy = reinterpret_cast<decltype(r.destroy)>(dlsym(lib, "rocblas_destroy_handle"));
            r.set_stream = reinterpret_cast<decltype(r.set_stream)>(dlsym(lib, "rocblas_set_stream"));
            r.sgemm = reinterpret_cast<decltype(r.sgemm)>(dlsym(lib, "rocblas_sgemm_strided_batched"));
            r.dgemm = reinterpret_cast<decltype(r.dgemm)>(dlsym(lib, "rocblas_dgemm_strided_batched"));
            r.ok = r.create && r.set_stream && r.sgemm && r.dgemm;
        }
    }
    return r.ok;
}

static RocBlas::Handle rocblas_handle_for(hipStream_t stream)
{
    int dev = 0;
    SIG_HIP(hipGetDevice(&dev));
    RocBlas::Handle& h = g_rocblas.handles[dev];
    if (!h && g_rocblas.create(&h) != 0) {
        h = nullptr;
        throw std::runtime_error("sig_backprop_cuda: rocblas_create_handle failed");
    }
    if (g_rocblas.set_stream(h, stream) != 0) throw std::runtime_error("sig_backprop_cuda: rocblas_set_stream failed");
    return h;
}

// rocBLAS strided-batched gemm as the library defines it (column-major): C[m x n] = op(A) op(B) + beta C
template <typename T>
static void gemm_col_major(RocBlas::Handle h, bool a_transposed, bool b_transposed, int m, int n, int k, const T* A, int lda,
                           int64_t sa, const T* B, int ldb, int64_t sb, T beta, T* C, int ldc, int64_t sc, int batches)
{
    const T alpha = T(1);
    constexpr int kNone = 111, kTrans = 112;
    int rc;
    if constexpr (sizeof(T) == 8)
        rc = g_rocblas.dgemm(h, a_transposed ? kTrans : kNone, b_transposed ? kTrans : kNone, m, n, k, &alpha, A, lda, sa, B, ldb, sb,
                             &beta, C, ldc, sc, batches);
    else
        rc = g_rocblas.sgemm(h, a_transposed ? kTrans : kNone, b_transposed ? kTrans : kNone, m, n, k, &alpha, A, lda, sa, B, ldb, sb,
                             &beta, C, ldc, sc, batches);
    if (rc != 0) throw std::runtime_error("rocBLAS gemm failed (status " + std::to_string(rc) + ")");
}

// gives the handles (and the device memory they hold) back; the library stays loaded.  Caller holds the workspace mutex.
static void rocblas_release() noexcept
{
    for (auto& kv : g_rocblas.handles) {
        if (!kv.second || !g_rocblas.destroy) continue;
        int cur = 0;
        if (hipGetDevice(&cur) == hipSuccess && hipSetDevice(kv.first) == hipSuccess) {
            (void)g_rocblas.destroy(kv.second);
            (void)hipSetDevice(cur);
        }
    }
    g_rocblas.handles.clear();
}

// row-major C[m x n] (ldc) = A[m x k] * op(B) + beta * C, batched; op(B) = B[k x n] or B^T with B[n x k].
// Column-major view: C^T[n x m] = op(B)^T A^T
template <typename T>
static void gemm_row_major(RocBlas::Handle h, bool b_transposed, int m, int n, int k, const T* A, int lda, int64_t sa,
                           const T* B, int ldb, int64_t sb, T beta, T* C, int ldc, int64_t sc, int batches)
{
    gemm_col_major<T>(h, b_transposed, false, n, m, k, B, ldb, sb, A, lda, sa, beta, C, ldc, sc, batches);
}

// ---- the scan ------------------------------------------------------------------------------------------------------
// Sums N values per lane (N = 16 or 32) over the 64 lanes of a wave with about N + 6 exchanges instead of 6 N: every
// exchange step halves the values a lane keeps (the partner takes the other half); plain steps finish the last value.
// On return lane l holds in v[0] the wave's total of value number l / (64 / N).
template <typename T, int N, int COUNT, int S>
__device__ __forceinline__ void wave_sum_many_step(T (&v)[N], int lane)
{
    if constexpr (COUNT > 1) {
        constexpr int half = COUNT / 2;
        const bool upper = (lane & S) != 0;
#pragma unroll
        for (int k = 0; k < half; ++k) {
            const T send = upper ? v[k] : v[k + half];
            const T keep = upper ? v[k + half] : v[k];
            v[k] = keep + __shfl_xor(send, S);
        }
        wave_sum_many_step<T, N, half, S / 2>(v, lane);
    } else if constexpr (S >= 1) {
        v[0] += __shfl_xor(v[0], S);
        wave_sum_many_step<T, N, 1, S / 2>(v, lane);
    }
}
template <typename T, int N>
__device__ __forceinline__ void wave_sum_many(T (&v)[N], int lane)
{
    static_assert(N == 16 || N == 32, "a power of two that divides the wave");
    wave_sum_many_step<T, N, N, 32>(v, lane);
}

// grid: x = column strips of 64 (j), y = paths of the chunk, z = sets of four row groups; wave w of a block carries the
// rows i = R g .. R g + R - 1 (g = 4 z + w) of its strip for all steps; waves never wait for each other.  buf:
// [path][L][d * d], holds Y on entry and V on exit.  dz ([path][L][d]) and r1 ([path][L][d]: what each step adds to the
// level-1 adjoint) receive the row and column sums through atomics (one instruction per wave and step each).
template <typename T>
__global__ __launch_bounds__(kBlock) void degree3_scan_kernel(
    const T* __restrict__ inc, const T* __restrict__ sig, const T* __restrict__ gsig, T* __restrict__ buf,
    T* __restrict__ dz, T* __restrict__ r1, int64_t L, int d, int64_t sig_stride, int scalar, int64_t first_path)
{
    constexpr int R = kDeg3RowsPerThread;
    const int lane = threadIdx.x & (kWave - 1), w = int(blockIdx.z) * kWavesPerBlock + int(threadIdx.x >> 6);
    const int j = blockIdx.x * kWave + lane;
    const bool jon = j < d;
    const int64_t pl = blockIdx.y, pg = first_path + pl;
    const T* z_rows = inc + (pg * (L + 2) + 1) * d;      // row t: increment of step t
    const T* S = sig + pg * sig_stride + scalar;
    const T* G = gsig + pg * sig_stride + scalar;
    T* Y = buf + pl * L * int64_t(d) * d;
    T* dzp = dz + pg * L * d;
    T* r1p = r1 + pg * L * d;
    const int i0 = w * R;
    if (i0 >= d) return;
    T a2[R], s2[R], s1[R], y[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int i = i0 + r;
        const bool on = jon && i < d;
        a2[r] = on ? G[d + i * d + j] : T(0);
        s2[r] = on ? S[d + i * d + j] : T(0);
        s1[r] = i < d ? S[i] : T(0);                      // level 1 of the state, rows of this wave (wave-uniform)
        y[r] = on ? Y[(L - 1) * int64_t(d) * d + i * d + j] : T(0);
    }
    // which total the lane holds after wave_sum_many: rows' dz term (values 0..15), rows' level-1 term (16..31)
    constexpr int kShare = kWave / (2 * R);       // lanes that end up with the same total
    const int mine = lane / kShare;
    const bool row_writer = lane % kShare == 0 && i0 + (mine & (R - 1)) < d;
    T* const row_dst = (mine < R ? dzp : r1p) + i0 + (mine & (R - 1));
    for (int64_t t = L - 1; t >= 0; --t) {
        const T* z = z_rows + t * d;
        T* Yt = Y + t * int64_t(d) * d;
        T yn[R];                                          // the next step's rows, in flight during this one
#pragma unroll
        for (int r = 0; r < R; ++r) yn[r] = (t > 0 && jon && i0 + r < d) ? Yt[(i0 + r) * d + j - int64_t(d) * d] : T(0);
        const T zj = jon ? z[j] : T(0);
        T cj = T(0);
        T sums[2 * R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int i = i0 + r;
            sums[r] = T(0);
            sums[R + r] = T(0);
            if (i < d) {                                  // wave-uniform
                const T zi = z[i];
                const T si = s1[r] - zi;                  // state before the step
                s1[r] = si;
                const T sp = s2[r] - (si + zi * T(0.5)) * zj;
                const T v = sp + (si * T(0.5) + zi * T(1.0 / 6.0)) * zj;
                if (jon) Yt[i * d + j] = v;
                cj = fmadd(a2[r], si + zi * T(0.5), cj);
                cj = fmadd(y[r], si * T(0.5) + zi * T(1.0 / 6.0), cj);
                const T az = a2[r] * zj, yz = y[r] * zj;  // idle lanes hold zeros
                sums[r] = az * T(0.5) + yz * T(1.0 / 6.0);
                sums[R + r] = az + yz * T(0.5);
                a2[r] += y[r];
                s2[r] = sp;
            }
            y[r] = yn[r];
        }
        if (jon) dev_add(dzp + t * d + j, cj);
        wave_sum_many(sums, lane);
        if (row_writer) dev_add(row_dst + t * d, sums[0]);
    }
}

// Forward: S3 = sum_t V_t (x) z_t = V^T Z with the same V_t = S2 + S1 (x) z_t / 2 + z_t (x) z_t / 6 (state before step
// t).  This scan walks the steps forwards, writes V ([path][L][d * d]) and leaves levels 1 and 2 (and the scalar term)
// in the output row; the product fills level 3.  Same grid as degree3_scan_kernel; no sums across lanes.
template <typename T>
__global__ __launch_bounds__(kBlock) void degree3_fwd_scan_kernel(const T* __restrict__ inc, T* __restrict__ buf,
                                                                  T* __restrict__ out, int64_t L, int d, int64_t out_stride,
                                                                  int scalar, int64_t first_path)
{
    constexpr int R = kDeg3RowsPerThread;
    const int lane = threadIdx.x & (kWave - 1), w = int(blockIdx.z) * kWavesPerBlock + int(threadIdx.x >> 6);
    const int j = blockIdx.x * kWave + lane;
    const bool jon = j < d;
    const int64_t pl = blockIdx.y, pg = first_path + pl;
    const T* z_rows = inc + (pg * (L + 2) + 1) * d;
    T* V = buf + pl * L * int64_t(d) * d;
    T* O = out + pg * out_stride + scalar;
    const int i0 = w * R;
    if (i0 >= d) return;
    T s2[R], s1[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        s2[r] = T(0);
        s1[r] = T(0);
    }
    T s1j = T(0);
    T zj = jon ? z_rows[j] : T(0);
    for (int64_t t = 0; t < L; ++t) {
        const T* z = z_rows + t * d;
        T* Vt = V + t * int64_t(d) * d;
        const T zn = (jon && t + 1 < L) ? z[d + j] : T(0);      // next step's increment, in flight during this one
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int i = i0 + r;
            if (i < d) {                                        // wave-uniform
                const T zi = z[i];
                if (jon) Vt[i * d + j] = fmadd(s1[r] * T(0.5) + zi * T(1.0 / 6.0), zj, s2[r]);
                s2[r] = fmadd(s1[r] + zi * T(0.5), zj, s2[r]);
                s1[r] += zi;
            }
        }
        s1j += zj;
        zj = zn;
    }
    if (jon) {
#pragma unroll
        for (int r = 0; r < R; ++r)
            if (i0 + r < d) O[d + (i0 + r) * d + j] = s2[r];
        if (i0 == 0) O[j] = s1j;
    }
    if (scalar && i0 == 0 && j == 0) out[pg * out_stride] = T(1);
}

// dz[t][m] += a1 after step t;  a1 runs backwards: a1 <- a1 + r1[t].  One thread per (path, m).
template <typename T>
__global__ __launch_bounds__(kBlock) void degree3_level1_kernel(const T* __restrict__ gsig, const T* __restrict__ r1,
                                                                T* __restrict__ dz, int64_t batch, int64_t L, int d,
                                                                int64_t sig_stride, int scalar)
{
    const int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x;
    if (e >= batch * d) return;
    const int64_t b = e / d;
    const int m = int(e - b * d);
    T a1 = gsig[b * sig_stride + scalar + m];
    for (int64_t t = L - 1; t >= 0; --t) {
        const int64_t at = (b * L + t) * d + m;
        dz[at] += a1;
        a1 += r1[at];
    }
}

}  // namespace sigamd
