// Degree 2 in closed form, on the matrix cores.
//
// With X_t the (augmented) path, z_t = X_{t+1} - X_t its increments and L their number, the Horner recursion of
// siglib/cpsig/cp_signature.h:464-499 unrolls at degree 2 to
//     S1 = X_L - X_0,      S2[a][b] = sum_t U_t[a] * z_t[b],      U_t = (X_t + X_{t+1}) / 2 - X_0,
// i.e. S2 = U^T Z: one (d x L) by (L x d) product per path, with no dependence between time steps.  Its pullback
// (the level-2 part of siglib/cpsig/cp_signature.h:1137-1187 summed over the sweep) is
//     dz_t = h + U_t (G2 - G2^T),      h = G1 + G2 S1,
// an (L x d) by (d x d) product with the antisymmetric part of the level-2 gradient.  Both run as MFMA 16x16x4 tiles
// (f32 and f64), operands built on the fly from the raw path: nothing is staged in HBM, lead-lag and time
// augmentation are evaluated per element.  Used for paths of many channels, where the sweep kernels' per-step work
// per lane is too small to run well.
#pragma once
#include <hip/hip_runtime.h>

#include "sig_kernels.h"

namespace sigamd {

// point t, channel c of the augmented path (siglib/cpsig/cp_path.h:46-62,262-279): lead-lag doubles the channels
// (first half lags: it moves on odd steps; second half leads: it moves on even steps), time is the last channel
template <typename T>
__device__ __forceinline__ T aug_point(const T* __restrict__ x, int64_t t, int c, int d_raw, int time_aug, int lead_lag,
                                       int d, T time_step)
{
    if (time_aug && c == d - 1) return mul_rn(T(t), time_step);
    if (!lead_lag) return x[t * d_raw + c];
    return c < d_raw ? x[(t >> 1) * d_raw + c] : x[((t + 1) >> 1) * d_raw + (c - d_raw)];
}

template <typename T>
struct Mfma16;
template <>
struct Mfma16<float> {
    typedef float Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row(int lk, int r) { return 4 * lk + r; }
};
template <>
struct Mfma16<double> {
    typedef double Acc __attribute__((ext_vector_type(4)));
    static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
    static __device__ __forceinline__ int row(int lk, int r) { return 4 * r + lk; }
};

// Tile conventions of the 16x16x4 instructions (checked on the device): lane l supplies A[i = l % 16][k = l / 16] and
// B[k = l / 16][j = l % 16] and receives, in component r of the accumulator, C[i][j = l % 16] with
// i = 4 * (l / 16) + r for f32 and i = 4 * r + l / 16 for f64 (Mfma16::row).
constexpr int kDeg2Cols = 4;     // 16-wide column tiles per wave
constexpr int kDeg2Unroll = 1;   // groups of 4 steps whose loads are in flight together (forward)

// Forward.  One wave per (path, time slice, 16-row tile a, group of kDeg2Cols column tiles b); slices of a path add
// into the output with atomics (the output is cleared first when there are several).
template <typename T>
__global__ __launch_bounds__(kBlock) void degree2_fwd_kernel(
    const T* __restrict__ path, T* __restrict__ out, int64_t batch, int64_t len_raw, int d_raw, int time_aug, int lead_lag,
    T time_step, int64_t out_stride, int scalar, int tiles, int col_groups, int slices, int64_t slice_len,
    int* __restrict__ nonfinite)
{
    using M = Mfma16<T>;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t per_path = int64_t(tiles) * col_groups * slices;
    const int64_t b = wave / per_path;
    if (b >= batch) return;
    int64_t w = wave - b * per_path;
    const int slice = int(w % slices);
    w /= slices;
    const int cg = int(w % col_groups);
    const int ta = int(w / col_groups);
    const T* x = path + b * len_raw * d_raw;
    T* o = out + b * out_stride + scalar;

    const int li = lane & 15, lk = lane >> 4;
    const int a = ta * 16 + li;                      // row channel this lane feeds
    const bool a_ok = a < d;
    const T x0a = a_ok ? aug_point(x, 0, a, d_raw, time_aug, lead_lag, d, time_step) : T(0);
    typename M::Acc acc[kDeg2Cols];
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) acc[j] = typename M::Acc{T(0), T(0), T(0), T(0)};

    const int nb = tiles - cg * kDeg2Cols < kDeg2Cols ? tiles - cg * kDeg2Cols : kDeg2Cols;     // column tiles in use
    const int64_t t_begin = int64_t(slice) * slice_len;
    const int64_t t_end = t_begin + slice_len < L ? t_begin + slice_len : L;
    // kDeg2Unroll groups of 4 steps per iteration: all their loads are issued before the first product
    for (int64_t t0 = t_begin; t0 < t_end; t0 += 4 * kDeg2Unroll) {
        T ua[kDeg2Unroll], zb[kDeg2Unroll][kDeg2Cols];
#pragma unroll
        for (int u = 0; u < kDeg2Unroll; ++u) {
            const int64_t t = t0 + 4 * u + lk;
            const bool t_ok = t < t_end;
            ua[u] = T(0);
            if (t_ok && a_ok) {
                const T p0 = aug_point(x, t, a, d_raw, time_aug, lead_lag, d, time_step);
                const T p1 = aug_point(x, t + 1, a, d_raw, time_aug, lead_lag, d, time_step);
                ua[u] = T(0.5) * (p0 + p1) - x0a;
            }
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) {
                const int c = (cg * kDeg2Cols + j) * 16 + li;
                zb[u][j] = T(0);
                if (t_ok && c < d)
                    zb[u][j] = aug_point(x, t + 1, c, d_raw, time_aug, lead_lag, d, time_step) -
                               aug_point(x, t, c, d_raw, time_aug, lead_lag, d, time_step);
            }
        }
#pragma unroll
        for (int u = 0; u < kDeg2Unroll; ++u) {
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j)
                if (j < nb) acc[j] = M::mma(ua[u], zb[u][j], acc[j]);
        }
    }

    T chk = T(0);
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) {
        const int c = (cg * kDeg2Cols + j) * 16 + li;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = ta * 16 + M::row(lk, r);
            if (row < d && c < d) {
                T* dst = o + d + int64_t(row) * d + c;
                if (slices > 1) dev_add(dst, acc[j][r]);
                else *dst = acc[j][r];
                chk = fmadd(acc[j][r], T(0), chk);
            }
        }
    }
    // level 1 and the scalar: written once per path
    if (cg == 0 && slice == 0 && lk == 0 && a_ok) {
        const T s1 = aug_point(x, L, a, d_raw, time_aug, lead_lag, d, time_step) - x0a;
        o[a] = s1;
        chk = fmadd(s1, T(0), chk);
        if (scalar && a == 0) o[-1] = T(1);
    }
    if (nonfinite && !(chk == T(0))) *nonfinite = 1;
}

// Forward, points staged through LDS.  A block serves one (path, time slice, group of four 16-row tiles, group of
// kDeg2Cols column tiles): its four waves own one row tile each and share the column group.  Per chunk of 4 * rq
// steps the block copies the points Y_t = X_t - X_0 of its 64 row channels and of its 64 column channels to LDS
// (coalesced reads of the path, every point read once per block; one slab when the two channel groups coincide).
// The four step indices k of a product stand for four contiguous runs of rq steps, so that a lane walks the rows of
// its run and forms U_t = (Y_t + Y_{t+1}) / 2 and z_t = Y_{t+1} - Y_t from the row it already holds and the next:
// one LDS read per operand and product.  Rows past the end of the slice repeat its last point (z = 0: no term).
// Slab rows are 80 words long and rq is odd, so that the four runs' rows fall into different banks.
constexpr int kDeg2Slab = 16 * kDeg2Cols;       // channels per slab (64)
constexpr int kDeg2SlabStride = kDeg2Slab + 16;
static_assert(kBlock % kDeg2Slab == 0 && kWavesPerBlock == kDeg2Cols, "staging assumes 4 waves and 64-channel slabs");

// MODE 0: any augmentation, a point's channels evaluated one by one.  MODE 1: neither lead-lag nor time augmentation
// (a point's channels are one contiguous row of the input).  MODE 2: such rows in 16-byte pieces (dimension a
// multiple of 16 bytes, aligned input), and the next chunk's pieces are loaded into registers before the products of
// the current one start, so that a block's loads and products overlap.
constexpr int kDeg2StageBatch = 8;      // staged rows whose loads a thread has in flight together
constexpr int kDeg2Prefetch = 9;        // 16-byte pieces a thread holds for the next chunk (MODE 2)
template <typename T>
struct Vec16;
template <>
struct Vec16<float> {
    typedef float type __attribute__((ext_vector_type(4)));
    static constexpr int n = 4;
};
template <>
struct Vec16<double> {
    typedef double type __attribute__((ext_vector_type(2)));
    static constexpr int n = 2;
};
// rows of a chunk that MODE 2 can hold in its registers
template <typename T>
constexpr int deg2_prefetch_rows() { return kDeg2Prefetch * (kBlock / (kDeg2Slab / Vec16<T>::n)); }

template <typename T, int MODE>
__global__ __launch_bounds__(kBlock) void degree2_fwd_staged_kernel(
    const T* __restrict__ path, T* __restrict__ out, int64_t batch, int64_t len_raw, int d_raw, int time_aug, int lead_lag,
    T time_step, int64_t out_stride, int scalar, int tiles, int col_groups, int slices, int64_t slice_len, int rq,
    int* __restrict__ nonfinite)
{
    using M = Mfma16<T>;
    extern __shared__ __align__(16) double lds_raw_d2[];
    constexpr bool PLAIN = MODE != 0;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int row_groups = (tiles + kWavesPerBlock - 1) / kWavesPerBlock;
    const int64_t per_path = int64_t(row_groups) * col_groups * slices;
    const int64_t b = int64_t(blockIdx.x) / per_path;          // grid = batch * per_path: every block has a path
    int64_t w = int64_t(blockIdx.x) - b * per_path;
    const int slice = int(w % slices);
    w /= slices;
    const int cg = int(w % col_groups);
    const int rg = int(w / col_groups);
    const int ta = rg * kWavesPerBlock + wave;                  // this wave's row tile
    const bool has_task = ta < tiles;
    const T* x = path + b * len_raw * d_raw;
    T* o = out + b * out_stride + scalar;
    const int rows = 4 * rq + 1;                                // points of a chunk
    T* lds_u = reinterpret_cast<T*>(lds_raw_d2);
    T* lds_z = rg == cg ? lds_u : lds_u + int64_t(rows) * kDeg2SlabStride;

    const int li = lane & 15, lk = lane >> 4;
    typename M::Acc acc[kDeg2Cols];
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) acc[j] = typename M::Acc{T(0), T(0), T(0), T(0)};
    const int nb = tiles - cg * kDeg2Cols < kDeg2Cols ? tiles - cg * kDeg2Cols : kDeg2Cols;

    // staging: a thread keeps one slab column and walks the chunk's rows
    const int sc_col = threadIdx.x % kDeg2Slab, sc_row0 = threadIdx.x / kDeg2Slab;
    const int cu = rg * kDeg2Slab + sc_col, cz = cg * kDeg2Slab + sc_col;
    const T x0u = cu < d ? aug_point(x, 0, cu, d_raw, time_aug, lead_lag, d, time_step) : T(0);
    const T x0z = cz < d ? aug_point(x, 0, cz, d_raw, time_aug, lead_lag, d, time_step) : T(0);

    const int64_t t_begin = int64_t(slice) * slice_len;
    const int64_t t_end = t_begin + slice_len < L ? t_begin + slice_len : L;
    auto point = [&](int64_t t, int c) {
        if constexpr (PLAIN) return x[t * d_raw + c];
        else return aug_point(x, t, c, d_raw, time_aug, lead_lag, d, time_step);
    };
    constexpr int kRowStep = kBlock / kDeg2Slab;
    // MODE 2: thread -> 16-byte piece `vcol` of the rows vrow0, vrow0 + kVecRows, ..
    using V = typename Vec16<T>::type;
    constexpr int kVecCols = kDeg2Slab / Vec16<T>::n, kVecRows = kBlock / kVecCols;
    const int vcol = int(threadIdx.x % kVecCols) * Vec16<T>::n, vrow0 = int(threadIdx.x / kVecCols);
    [[maybe_unused]] V pfu[kDeg2Prefetch], pfz[kDeg2Prefetch], x0uv = V(T(0)), x0zv = V(T(0));
    [[maybe_unused]] const bool vu_ok = rg * kDeg2Slab + vcol < d, vz_ok = rg != cg && cg * kDeg2Slab + vcol < d;
    [[maybe_unused]] auto fetch = [&](int64_t t0) {
#pragma unroll
        for (int k = 0; k < kDeg2Prefetch; ++k) {
            const int r = vrow0 + kVecRows * k;
            const int64_t t = t0 + r < t_end ? t0 + r : t_end;
            pfu[k] = vu_ok ? *reinterpret_cast<const V*>(x + t * d_raw + rg * kDeg2Slab + vcol) : V(T(0));
            pfz[k] = vz_ok ? *reinterpret_cast<const V*>(x + t * d_raw + cg * kDeg2Slab + vcol) : V(T(0));
        }
    };
    if constexpr (MODE == 2) {
        if (vu_ok) x0uv = *reinterpret_cast<const V*>(x + rg * kDeg2Slab + vcol);
        if (vz_ok) x0zv = *reinterpret_cast<const V*>(x + cg * kDeg2Slab + vcol);
        fetch(t_begin);
    }
    for (int64_t t0 = t_begin; t0 < t_end; t0 += 4 * rq) {
        __syncthreads();        // the previous chunk has been consumed
        if constexpr (MODE == 2) {
#pragma unroll
            for (int k = 0; k < kDeg2Prefetch; ++k) {
                const int r = vrow0 + kVecRows * k;
                if (r < rows) {
                    *reinterpret_cast<V*>(lds_u + r * kDeg2SlabStride + vcol) = pfu[k] - x0uv;
                    if (rg != cg) *reinterpret_cast<V*>(lds_z + r * kDeg2SlabStride + vcol) = pfz[k] - x0zv;
                }
            }
        } else {
            for (int r0 = sc_row0; r0 < rows; r0 += kRowStep * kDeg2StageBatch) {
                T vu[kDeg2StageBatch], vz[kDeg2StageBatch];
#pragma unroll
                for (int k = 0; k < kDeg2StageBatch; ++k) {
                    const int r = r0 + kRowStep * k;
                    const int64_t t = t0 + r < t_end ? t0 + r : t_end;
                    vu[k] = cu < d ? point(t, cu) : T(0);
                    vz[k] = (rg != cg && cz < d) ? point(t, cz) : T(0);
                }
#pragma unroll
                for (int k = 0; k < kDeg2StageBatch; ++k) {
                    const int r = r0 + kRowStep * k;
                    if (r < rows) {
                        lds_u[r * kDeg2SlabStride + sc_col] = vu[k] - x0u;
                        if (rg != cg) lds_z[r * kDeg2SlabStride + sc_col] = vz[k] - x0z;
                    }
                }
            }
        }
        __syncthreads();
        if constexpr (MODE == 2)
            if (t0 + 4 * rq < t_end) fetch(t0 + 4 * rq);
        if (has_task) {
            const T* pu = lds_u + lk * rq * kDeg2SlabStride + wave * 16 + li;
            const T* pz = lds_z + lk * rq * kDeg2SlabStride + li;
            // all kDeg2Cols column tiles, in use or not (channels past the last hold zeros): no branch in the loop
            // the rows r and r + 1 are in registers while row r + 2 is on its way from LDS
            T u0 = pu[0], u1 = pu[kDeg2SlabStride], z0[kDeg2Cols], z1[kDeg2Cols];
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) {
                z0[j] = pz[j * 16];
                z1[j] = pz[kDeg2SlabStride + j * 16];
            }
            for (int r = 1; r <= rq; ++r) {
                const int rn = r < rq ? r + 1 : r;
                const T u2 = pu[rn * kDeg2SlabStride];
                T z2[kDeg2Cols];
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) z2[j] = pz[rn * kDeg2SlabStride + j * 16];
                const T ua = T(0.5) * (u0 + u1);
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) acc[j] = M::mma(ua, z1[j] - z0[j], acc[j]);
                u0 = u1;
                u1 = u2;
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) {
                    z0[j] = z1[j];
                    z1[j] = z2[j];
                }
            }
        }
    }
    if (!has_task) return;

    T chk = T(0);
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) {
        const int c = (cg * kDeg2Cols + j) * 16 + li;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int row = ta * 16 + M::row(lk, r);
            if (row < d && c < d) {
                T* dst = o + d + int64_t(row) * d + c;
                if (slices > 1) dev_add(dst, acc[j][r]);
                else *dst = acc[j][r];
                chk = fmadd(acc[j][r], T(0), chk);
            }
        }
    }
    const int a = ta * 16 + li;
    if (cg == 0 && slice == 0 && lk == 0 && a < d) {
        const T s1 = aug_point(x, L, a, d_raw, time_aug, lead_lag, d, time_step) - aug_point(x, 0, a, d_raw, time_aug, lead_lag, d, time_step);
        o[a] = s1;
        chk = fmadd(s1, T(0), chk);
        if (scalar && a == 0) o[-1] = T(1);
    }
    if (nonfinite && !(chk == T(0))) *nonfinite = 1;
}

// Slices of one path accumulate with atomics: a sum of finite parts can still overflow, so the flag is set from the
// finished rows.
template <typename T>
__global__ __launch_bounds__(kBlock) void finite_rows_kernel(const T* __restrict__ rows, int64_t total, int* __restrict__ nonfinite)
{
    T chk = T(0);
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock)
        chk = fmadd(rows[e], T(0), chk);
    if (!(chk == T(0))) *nonfinite = 1;
}

// h[b][c] = G1[c] + sum_e G2[c][e] * S1[e]: one wave per (path, c), its lanes a coalesced walk along the row
template <typename T>
__global__ __launch_bounds__(kBlock) void degree2_h_kernel(
    const T* __restrict__ path, const T* __restrict__ gsig, T* __restrict__ h, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, T time_step, int64_t sig_stride, int scalar)
{
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t waves = int64_t(gridDim.x) * kWavesPerBlock;
    for (int64_t e = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); e < batch * d; e += waves) {
        const int64_t b = e / d;
        const int c = int(e - b * d);
        const T* x = path + b * len_raw * d_raw;
        const T* g = gsig + b * sig_stride + scalar;
        const T* grow = g + d + int64_t(c) * d;
        T s0 = T(0);
        for (int k = lane; k < d; k += kWave) {
            const T v = aug_point(x, L, k, d_raw, time_aug, lead_lag, d, time_step) - aug_point(x, 0, k, d_raw, time_aug, lead_lag, d, time_step);
            s0 = fmadd(grow[k], v, s0);
        }
        s0 = wave_sum(s0);
        if (lane == 0) h[e] = g[c] + s0;
    }
}

// Backward: dz[b][t][c] = h[b][c] + sum_a U_t[a] * (G2[a][c] - G2[c][a]).  One wave per (path, 16 steps, group of
// kDeg2Cols column tiles); the product runs over the channels a in steps of 4.
template <typename T>
__global__ __launch_bounds__(kBlock) void degree2_bwd_kernel(
    const T* __restrict__ path, const T* __restrict__ gsig, const T* __restrict__ h, T* __restrict__ dz, int64_t batch,
    int64_t len_raw, int d_raw, int time_aug, int lead_lag, T time_step, int64_t sig_stride, int scalar, int64_t time_tiles,
    int col_groups)
{
    using M = Mfma16<T>;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wave = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    const int64_t per_path = time_tiles * col_groups;
    const int64_t b = wave / per_path;
    if (b >= batch) return;
    const int64_t w = wave - b * per_path;
    const int cg = int(w % col_groups);
    const int64_t tt = w / col_groups;
    const T* x = path + b * len_raw * d_raw;
    const T* g2 = gsig + b * sig_stride + scalar + d;

    const int li = lane & 15, lk = lane >> 4;
    const int tiles = (d + 15) / 16;
    const int nb = tiles - cg * kDeg2Cols < kDeg2Cols ? tiles - cg * kDeg2Cols : kDeg2Cols;     // column tiles in use
    const int64_t t = tt * 16 + li;                  // step this lane feeds as a row of U
    const bool t_ok = t < L;
    typename M::Acc acc[kDeg2Cols];
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) acc[j] = typename M::Acc{T(0), T(0), T(0), T(0)};

    for (int a0 = 0; a0 < d; a0 += 4) {
        const int a = a0 + lk;
        const bool a_ok = a < d;
        T ua = T(0);
        if (t_ok && a_ok) {
            const T p0 = aug_point(x, t, a, d_raw, time_aug, lead_lag, d, time_step);
            const T p1 = aug_point(x, t + 1, a, d_raw, time_aug, lead_lag, d, time_step);
            ua = T(0.5) * (p0 + p1) - aug_point(x, 0, a, d_raw, time_aug, lead_lag, d, time_step);
        }
#pragma unroll
        for (int j = 0; j < kDeg2Cols; ++j) {
            const int c = (cg * kDeg2Cols + j) * 16 + li;
            T anti = T(0);
            if (a_ok && c < d) anti = g2[int64_t(a) * d + c] - g2[int64_t(c) * d + a];
            if (j < nb) acc[j] = M::mma(ua, anti, acc[j]);
        }
    }

#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) {
        const int c = (cg * kDeg2Cols + j) * 16 + li;
        if (c >= d) continue;
        const T hc = h[b * d + c];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t row = tt * 16 + M::row(lk, r);
            if (row < L) dz[(b * L + row) * d + c] = acc[j][r] + hc;
        }
    }
}

// anti[b][a][c] = G2[a][c] - G2[c][a]: written once per call so that the staged backward reads it row-wise
template <typename T>
__global__ __launch_bounds__(kBlock) void degree2_anti_kernel(
    const T* __restrict__ gsig, T* __restrict__ anti, int64_t batch, int d, int64_t sig_stride, int scalar)
{
    const int64_t dd = int64_t(d) * d;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < batch * dd; e += int64_t(gridDim.x) * kBlock) {
        const int64_t b = e / dd;
        const int64_t r = e - b * dd;
        const int a = int(r / d), c = int(r - int64_t(a) * d);
        const T* g2 = gsig + b * sig_stride + scalar + d;
        anti[e] = g2[r] - g2[int64_t(c) * d + a];
    }
}

// Backward, operands staged through LDS.  A block serves one (path, 64 steps, group of kDeg2Cols column tiles): its
// four waves own 16 steps each and share the column group.  The product runs over the channels a in chunks of 64: per
// chunk the block writes U[64 steps][64 channels] and anti[64 channels][64 columns] to LDS, then every wave feeds its
// products from there.  Row strides are chosen so that fragment reads are bank-conflict free: the U fragment walks
// rows with its 16 lanes (stride 66 words f32 / 65 f64), the anti fragment walks columns (stride 80).
template <typename T>
__global__ __launch_bounds__(kBlock) void degree2_bwd_staged_kernel(
    const T* __restrict__ path, const T* __restrict__ anti, const T* __restrict__ h, T* __restrict__ dz, int64_t batch,
    int64_t len_raw, int d_raw, int time_aug, int lead_lag, T time_step, int64_t time_groups, int col_groups)
{
    using M = Mfma16<T>;
    extern __shared__ double lds_raw_d2b[];
    constexpr int SU = sizeof(T) == 8 ? 65 : 66;
    constexpr int SA = kDeg2SlabStride;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    T* lds_u = reinterpret_cast<T*>(lds_raw_d2b);
    T* lds_a = lds_u + kDeg2Slab * SU;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x >> 6;
    const int64_t per_path = time_groups * col_groups;
    const int64_t b = int64_t(blockIdx.x) / per_path;           // grid = batch * per_path
    const int64_t w = int64_t(blockIdx.x) - b * per_path;
    const int cg = int(w % col_groups);
    const int64_t tg = w / col_groups;
    const T* x = path + b * len_raw * d_raw;
    const T* an = anti + b * int64_t(d) * d;

    const int li = lane & 15, lk = lane >> 4;
    const int tiles = (d + 15) / 16;
    const int nb = tiles - cg * kDeg2Cols < kDeg2Cols ? tiles - cg * kDeg2Cols : kDeg2Cols;
    typename M::Acc acc[kDeg2Cols];
#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) acc[j] = typename M::Acc{T(0), T(0), T(0), T(0)};

    const int sc_col = threadIdx.x % kDeg2Slab, sc_row0 = threadIdx.x / kDeg2Slab;
    const int64_t t_base = tg * kDeg2Slab;
    for (int a0 = 0; a0 < d; a0 += kDeg2Slab) {
        __syncthreads();        // the previous chunk has been consumed
        {
            // U: rows are steps, columns channels a0 + sc_col
            const int a = a0 + sc_col;
            const T x0 = a < d ? aug_point(x, 0, a, d_raw, time_aug, lead_lag, d, time_step) : T(0);
            for (int r = sc_row0; r < kDeg2Slab; r += kBlock / kDeg2Slab) {
                const int64_t t = t_base + r;
                T u = T(0);
                if (t < L && a < d)
                    u = T(0.5) * (aug_point(x, t, a, d_raw, time_aug, lead_lag, d, time_step) +
                                  aug_point(x, t + 1, a, d_raw, time_aug, lead_lag, d, time_step)) - x0;
                lds_u[r * SU + sc_col] = u;
            }
            // anti: rows are channels a0 + r, columns cg * 64 + sc_col
            const int c = cg * kDeg2Slab + sc_col;
            for (int r = sc_row0; r < kDeg2Slab; r += kBlock / kDeg2Slab) {
                const int aa = a0 + r;
                lds_a[r * SA + sc_col] = (aa < d && c < d) ? an[int64_t(aa) * d + c] : T(0);
            }
        }
        __syncthreads();
        const T* pu = lds_u + (wave * 16 + li) * SU + lk;
        const T* pa = lds_a + lk * SA + li;
        const int kmax = d - a0 < kDeg2Slab ? d - a0 : kDeg2Slab;
        for (int k0 = 0; k0 < kmax; k0 += 4) {
            const T ua = pu[k0];
            T ab[kDeg2Cols];
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) ab[j] = j < nb ? pa[k0 * SA + j * 16] : T(0);
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j)
                if (j < nb) acc[j] = M::mma(ua, ab[j], acc[j]);
        }
    }

#pragma unroll
    for (int j = 0; j < kDeg2Cols; ++j) {
        const int c = (cg * kDeg2Cols + j) * 16 + li;
        if (c >= d) continue;
        const T hc = h[b * d + c];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int64_t row = t_base + wave * 16 + M::row(lk, r);
            if (row < L) dz[(b * L + row) * d + c] = acc[j][r] + hc;
        }
    }
}

// Backward for at most 64 (augmented) channels, one launch.  A block serves a run of output rows of one path, 64 rows
// at a time: four waves of 16 rows each, all kDeg2Cols column tiles.  The antisymmetric part of the level-2 gradient
// is built once per block (G2 copied to LDS with coalesced loads, then every lane keeps its 16 x kDeg2Cols fragment
// values in registers for the whole run), and h = G1 + G2 S1 is formed in the block as well.  The product's k index
// stands for the channel lk * 16 + kk, so that a lane reads its 16 operands of a row as four 16-byte pieces.
// MODE 0: any augmentation; output rows are the increments' gradients dz_t = h + U_t A, t < L.
// MODE 1 / 2 (plain paths; 2: input rows in 16-byte pieces, next 64 rows prefetched into registers): the rows are the
// path's gradient itself, out_t = dz_{t-1} - dz_t = (Y_{t-1} - Y_{t+1}) / 2 A for 0 < t < L, out_0 = -dz_0,
// out_L = dz_{L-1}: with Y_{-1} = Y_0 = 0 and Y_{L+1} = -Y_L the same operand form serves every row, and only the
// two end rows see h.
constexpr int kDeg2BwdRows = 64;                    // output rows per chunk
constexpr int kDeg2BwdStride = kDeg2Slab + 4;       // LDS row of points: 16-byte pieces of neighbouring rows in different banks
constexpr int kDeg2GStride = kDeg2Slab + 1;         // LDS row of G2: a column walk changes bank
template <typename T>
constexpr size_t deg2_bwd_lds_bytes()
{
    return (size_t(kDeg2BwdRows + 2) * kDeg2BwdStride + size_t(kDeg2Slab) * kDeg2GStride + 2 * kDeg2Slab) * sizeof(T);
}

// registers for three (f32) resp. two (f64) blocks per CU: a block's phases (copy to LDS, products, stores) do not
// overlap with each other, only with those of its neighbours
template <typename T, int MODE>
__global__ __launch_bounds__(kBlock, sizeof(T) == 8 ? 2 : 3) void degree2_bwd_rows_kernel(
    const T* __restrict__ path, const T* __restrict__ gsig, T* __restrict__ outp, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, T time_step, int64_t sig_stride, int scalar, int parts, int64_t part_rows)
{
    using M = Mfma16<T>;
    using V = typename Vec16<T>::type;
    constexpr int VN = Vec16<T>::n;
    constexpr bool DIRECT = MODE != 0;
    constexpr int HI = DIRECT ? 2 : 1;              // the operand of row i combines the staged rows i and i + HI
    extern __shared__ __align__(16) double lds_raw_d2r[];
    T* Ys = reinterpret_cast<T*>(lds_raw_d2r);
    T* Gs = Ys + (kDeg2BwdRows + 2) * kDeg2BwdStride;
    T* hb = Gs + kDeg2Slab * kDeg2GStride;
    T* s1 = hb + kDeg2Slab;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int64_t out_rows = DIRECT ? L + 1 : L;
    const int64_t b = int64_t(blockIdx.x) / parts;
    const int part = int(int64_t(blockIdx.x) - b * parts);
    const int64_t row_begin = int64_t(part) * part_rows;
    const int64_t row_end = row_begin + part_rows < out_rows ? row_begin + part_rows : out_rows;
    if (row_begin >= row_end) return;
    const T* x = path + b * len_raw * d_raw;
    const T* g1 = gsig + b * sig_stride + scalar;
    const T* g2 = g1 + d;
    T* o = outp + b * out_rows * d;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int li = lane & 15, lk = lane >> 4;
    auto point = [&](int64_t t, int c) {
        if constexpr (DIRECT) return x[t * d_raw + c];
        else return aug_point(x, t, c, d_raw, time_aug, lead_lag, d, time_step);
    };
    // staged row r of the chunk at `base`: the point base + r - (DIRECT ? 1 : 0), as Y = X - X_0
    //   before the path: 0;  past it: -Y_L once (DIRECT), then 0
    constexpr int kVecCols = kDeg2Slab / VN, kVecRows = kBlock / kVecCols;
    constexpr int kPf = (kDeg2BwdRows + 2 + kVecRows - 1) / kVecRows;
    const int vcol = (tid % kVecCols) * VN, vrow0 = tid / kVecCols;
    [[maybe_unused]] V pf[kPf], x0v = V(T(0));
    [[maybe_unused]] const bool v_ok = vcol < d;
    [[maybe_unused]] auto fetch = [&](int64_t base) {
#pragma unroll
        for (int k = 0; k < kPf; ++k) {
            const int64_t t = base + vrow0 + kVecRows * k - 1;
            const int64_t tc = t < 0 ? 0 : (t > L ? L : t);
            pf[k] = v_ok ? *reinterpret_cast<const V*>(x + tc * d_raw + vcol) : V(T(0));
        }
    };
    if constexpr (MODE == 2) {
        if (v_ok) x0v = *reinterpret_cast<const V*>(x + vcol);
        fetch(row_begin);
    }
    // G2 and S1 to LDS
    for (int e = tid; e < kDeg2Slab * kDeg2Slab; e += kBlock) {
        const int a = e / kDeg2Slab, c = e % kDeg2Slab;
        Gs[a * kDeg2GStride + c] = (a < d && c < d) ? g2[int64_t(a) * d + c] : T(0);
    }
    if (tid < kDeg2Slab) s1[tid] = tid < d ? point(L, tid) - point(0, tid) : T(0);
    __syncthreads();
    // fragments of A = G2 - G2^T: lane (li, lk) supplies A[lk * 16 + kk][16 j + li].  They are the same for the four
    // waves: the first one builds them and, once h is done, puts them in place of G2, in the order the products read
    T bf[16][kDeg2Cols];
    if (wave == 0) {
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) {
                const int a = lk * 16 + kk, c = 16 * j + li;
                bf[kk][j] = T(0.5) * (Gs[a * kDeg2GStride + c] - Gs[c * kDeg2GStride + a]);     // the operands' 1/2 sits here
            }
        }
    } else if (wave == 1) {
        T sum[4] = {lane < d ? g1[lane] : T(0), T(0), T(0), T(0)};
#pragma unroll
        for (int e = 0; e < kDeg2Slab; e += 4) {
#pragma unroll
            for (int q = 0; q < 4; ++q) sum[q] = fmadd(Gs[lane * kDeg2GStride + e + q], s1[e + q], sum[q]);
        }
        hb[lane] = (sum[0] + sum[1]) + (sum[2] + sum[3]);
    }
    __syncthreads();
    T* Bf = Gs;                                     // [kk][lane][j]
    if (wave == 0) {
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) Bf[(kk * kWave + lane) * kDeg2Cols + j] = bf[kk][j];
        }
    }
    const int sc_col = tid % kDeg2Slab, sc_row0 = tid / kDeg2Slab;
    const T x0s = (MODE != 2 && sc_col < d) ? point(0, sc_col) : T(0);

    for (int64_t base = row_begin; base < row_end; base += kDeg2BwdRows) {
        __syncthreads();        // the chunk before has been consumed (first pass: hb is complete)
        if constexpr (MODE == 2) {
#pragma unroll
            for (int k = 0; k < kPf; ++k) {
                const int r = vrow0 + kVecRows * k;
                const int64_t t = base + r - 1;
                if (r < kDeg2BwdRows + 2) {
                    V v = pf[k] - x0v;
                    if (t < 0 || t > L + 1) v = V(T(0));
                    else if (t == L + 1) v = -v;
                    *reinterpret_cast<V*>(Ys + r * kDeg2BwdStride + vcol) = v;
                }
            }
        } else {
            constexpr int kRowStep = kBlock / kDeg2Slab;
            for (int r0 = sc_row0; r0 < kDeg2BwdRows + 2; r0 += kRowStep * kDeg2StageBatch) {
                T v[kDeg2StageBatch];
#pragma unroll
                for (int k = 0; k < kDeg2StageBatch; ++k) {
                    const int64_t t = base + r0 + kRowStep * k - (DIRECT ? 1 : 0);
                    const int64_t tc = t < 0 ? 0 : (t > L ? L : t);
                    v[k] = sc_col < d ? point(tc, sc_col) - x0s : T(0);
                    if (t < 0 || t > L + 1 || (!DIRECT && t > L)) v[k] = T(0);
                    else if (t == L + 1) v[k] = -v[k];
                }
#pragma unroll
                for (int k = 0; k < kDeg2StageBatch; ++k) {
                    const int r = r0 + kRowStep * k;
                    if (r < kDeg2BwdRows + 2) Ys[r * kDeg2BwdStride + sc_col] = v[k];
                }
            }
        }
        __syncthreads();
        if constexpr (MODE == 2)
            if (base + kDeg2BwdRows < row_end) fetch(base + kDeg2BwdRows);
        if (base + 16 * wave < row_end) {
            const T* lo = Ys + (16 * wave + li) * kDeg2BwdStride + lk * 16;
            const T* hi = lo + HI * kDeg2BwdStride;
            T u[16];
#pragma unroll
            for (int q = 0; q < 16 / VN; ++q) {
                const V a = *reinterpret_cast<const V*>(lo + q * VN), c = *reinterpret_cast<const V*>(hi + q * VN);
#pragma unroll
                for (int e = 0; e < VN; ++e) u[q * VN + e] = DIRECT ? a[e] - c[e] : a[e] + c[e];
            }
            typename M::Acc acc[kDeg2Cols];
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) acc[j] = typename M::Acc{T(0), T(0), T(0), T(0)};
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
                T bq[kDeg2Cols];
#pragma unroll
                for (int q = 0; q < kDeg2Cols / VN; ++q) {
                    const V v = *reinterpret_cast<const V*>(Bf + (kk * kWave + lane) * kDeg2Cols + q * VN);
#pragma unroll
                    for (int e = 0; e < VN; ++e) bq[q * VN + e] = v[e];
                }
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) acc[j] = M::mma(u[kk], bq[j], acc[j]);
            }
#pragma unroll
            for (int j = 0; j < kDeg2Cols; ++j) {
                const int c = 16 * j + li;
                if (c >= d) continue;
                const T hc = hb[c];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t row = base + 16 * wave + M::row(lk, r);
                    if (row < row_end) {
                        T v = acc[j][r];
                        if constexpr (DIRECT) v += row == 0 ? -hc : (row == L ? hc : T(0));
                        else v += hc;
                        o[row * d + c] = v;
                    }
                }
            }
        }
    }
}

// Backward for more than 64 channels.  A block serves (path, run of up to RC x 64 output rows, 64 columns) and keeps
// the RC x kDeg2Cols accumulator tiles of all its rows in registers while it walks the channels 64 at a time: per
// channel chunk it builds the fragments of the 64 x 64 block of (G2 - G2^T) / 2 once (the two blocks of G2 pass
// through one LDS tile, one after the other) and then, for each 64-row chunk, copies the points' channels of that
// chunk to LDS and runs the products as degree2_bwd_rows_kernel does.  h = G1 + G2 S1 comes from degree2_h_kernel.
// MODE as in degree2_bwd_rows_kernel.
template <typename T>
constexpr int deg2_wide_chunks() { return sizeof(T) == 8 ? 2 : 4; }

template <typename T, int MODE>
__global__ __launch_bounds__(kBlock, 2) void degree2_bwd_wide_kernel(
    const T* __restrict__ path, const T* __restrict__ gsig, const T* __restrict__ h, T* __restrict__ outp, int64_t batch,
    int64_t len_raw, int d_raw, int time_aug, int lead_lag, T time_step, int64_t sig_stride, int scalar, int parts,
    int col_groups)
{
    using M = Mfma16<T>;
    using V = typename Vec16<T>::type;
    constexpr int VN = Vec16<T>::n;
    constexpr bool DIRECT = MODE != 0;
    constexpr int HI = DIRECT ? 2 : 1;
    constexpr int RC = deg2_wide_chunks<T>();
    extern __shared__ __align__(16) double lds_raw_d2w[];
    T* Ys = reinterpret_cast<T*>(lds_raw_d2w);
    T* Gs = Ys + (kDeg2BwdRows + 2) * kDeg2BwdStride;
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int64_t out_rows = DIRECT ? L + 1 : L;
    const int64_t per_path = int64_t(parts) * col_groups;
    const int64_t b = int64_t(blockIdx.x) / per_path;
    const int64_t w = int64_t(blockIdx.x) - b * per_path;
    const int cg = int(w % col_groups);
    const int64_t row_begin = (w / col_groups) * (RC * kDeg2BwdRows);
    const int64_t row_end = row_begin + RC * kDeg2BwdRows < out_rows ? row_begin + RC * kDeg2BwdRows : out_rows;
    if (row_begin >= row_end) return;
    const T* x = path + b * len_raw * d_raw;
    const T* g2 = gsig + b * sig_stride + scalar + d;
    T* o = outp + b * out_rows * d;
    const int tid = threadIdx.x, lane = tid & (kWave - 1), wave = tid >> 6;
    const int li = lane & 15, lk = lane >> 4;
    const int c0 = cg * kDeg2Slab;
    auto point = [&](int64_t t, int c) {
        if constexpr (DIRECT) return x[t * d_raw + c];
        else return aug_point(x, t, c, d_raw, time_aug, lead_lag, d, time_step);
    };
    constexpr int kVecCols = kDeg2Slab / VN, kVecRows = kBlock / kVecCols;
    const int vcol = (tid % kVecCols) * VN, vrow0 = tid / kVecCols;
    const int sc_col = tid % kDeg2Slab, sc_row0 = tid / kDeg2Slab;

    typename M::Acc acc[RC][kDeg2Cols];
#pragma unroll
    for (int rc = 0; rc < RC; ++rc) {
#pragma unroll
        for (int j = 0; j < kDeg2Cols; ++j) acc[rc][j] = typename M::Acc{T(0), T(0), T(0), T(0)};
    }

    for (int a0 = 0; a0 < d; a0 += kDeg2Slab) {
        // fragments of the block (a0 .., c0 ..) of (G2 - G2^T) / 2
        __syncthreads();        // the products of the channel chunk before are done with Gs and Ys
        for (int e = tid; e < kDeg2Slab * kDeg2Slab; e += kBlock) {
            const int a = a0 + e / kDeg2Slab, c = c0 + e % kDeg2Slab;
            Gs[(e / kDeg2Slab) * kDeg2GStride + e % kDeg2Slab] = (a < d && c < d) ? g2[int64_t(a) * d + c] : T(0);
        }
        __syncthreads();
        T bf[16][kDeg2Cols];
        if (wave == 0) {
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) bf[kk][j] = Gs[(lk * 16 + kk) * kDeg2GStride + 16 * j + li];
            }
        }
        __syncthreads();
        for (int e = tid; e < kDeg2Slab * kDeg2Slab; e += kBlock) {
            const int c = c0 + e / kDeg2Slab, a = a0 + e % kDeg2Slab;
            Gs[(e / kDeg2Slab) * kDeg2GStride + e % kDeg2Slab] = (a < d && c < d) ? g2[int64_t(c) * d + a] : T(0);
        }
        __syncthreads();
        if (wave == 0) {
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j)
                    bf[kk][j] = T(0.5) * (bf[kk][j] - Gs[(16 * j + li) * kDeg2GStride + lk * 16 + kk]);
            }
        }
        __syncthreads();
        T* Bf = Gs;                                     // [kk][lane][j]
        if (wave == 0) {
#pragma unroll
            for (int kk = 0; kk < 16; ++kk) {
#pragma unroll
                for (int j = 0; j < kDeg2Cols; ++j) Bf[(kk * kWave + lane) * kDeg2Cols + j] = bf[kk][j];
            }
        }
#pragma unroll
        for (int rc = 0; rc < RC; ++rc) {
            const int64_t base = row_begin + int64_t(rc) * kDeg2BwdRows;
            if (base >= row_end) continue;          // block-uniform
            __syncthreads();    // the chunk before has been consumed (first pass: Bf is complete)
            if constexpr (MODE == 2) {
                const bool v_ok = a0 + vcol < d;
                const V x0v = v_ok ? *reinterpret_cast<const V*>(x + a0 + vcol) : V(T(0));
                for (int r = vrow0; r < kDeg2BwdRows + 2; r += kVecRows) {
                    const int64_t t = base + r - 1;
                    const int64_t tc = t < 0 ? 0 : (t > L ? L : t);
                    V v = v_ok ? *reinterpret_cast<const V*>(x + tc * d_raw + a0 + vcol) - x0v : V(T(0));
                    if (t < 0 || t > L + 1) v = V(T(0));
                    else if (t == L + 1) v = -v;
                    *reinterpret_cast<V*>(Ys + r * kDeg2BwdStride + vcol) = v;
                }
            } else {
                constexpr int kRowStep = kBlock / kDeg2Slab;
                const int a = a0 + sc_col;
                const T x0s = a < d ? point(0, a) : T(0);
                for (int r0 = sc_row0; r0 < kDeg2BwdRows + 2; r0 += kRowStep * kDeg2StageBatch) {
                    T v[kDeg2StageBatch];
#pragma unroll
                    for (int k = 0; k < kDeg2StageBatch; ++k) {
                        const int64_t t = base + r0 + kRowStep * k - (DIRECT ? 1 : 0);
                        const int64_t tc = t < 0 ? 0 : (t > L ? L : t);
                        v[k] = a < d ? point(tc, a) - x0s : T(0);
                        if (t < 0 || t > L + 1 || (!DIRECT && t > L)) v[k] = T(0);
                        else if (t == L + 1) v[k] = -v[k];
                    }
#pragma unroll
                    for (int k = 0; k < kDeg2StageBatch; ++k) {
                        const int r = r0 + kRowStep * k;
                        if (r < kDeg2BwdRows + 2) Ys[r * kDeg2BwdStride + sc_col] = v[k];
                    }
                }
            }
            __syncthreads();
            if (base + 16 * wave < row_end) {
                const T* lo = Ys + (16 * wave + li) * kDeg2BwdStride + lk * 16;
                const T* hi = lo + HI * kDeg2BwdStride;
                T u[16];
#pragma unroll
                for (int q = 0; q < 16 / VN; ++q) {
                    const V va = *reinterpret_cast<const V*>(lo + q * VN), vc = *reinterpret_cast<const V*>(hi + q * VN);
#pragma unroll
                    for (int e = 0; e < VN; ++e) u[q * VN + e] = DIRECT ? va[e] - vc[e] : va[e] + vc[e];
                }
#pragma unroll
                for (int kk = 0; kk < 16; ++kk) {
                    T bq[kDeg2Cols];
#pragma unroll
                    for (int q = 0; q < kDeg2Cols / VN; ++q) {
                        const V v = *reinterpret_cast<const V*>(Bf + (kk * kWave + lane) * kDeg2Cols + q * VN);
#pragma unroll
                        for (int e = 0; e < VN; ++e) bq[q * VN + e] = v[e];
                    }
#pragma unroll
                    for (int j = 0; j < kDeg2Cols; ++j) acc[rc][j] = M::mma(u[kk], bq[j], acc[rc][j]);
                }
            }
        }
    }

#pragma unroll
    for (int rc = 0; rc < RC; ++rc) {
        const int64_t base = row_begin + int64_t(rc) * kDeg2BwdRows;
#pragma unroll
        for (int j = 0; j < kDeg2Cols; ++j) {
            const int c = c0 + 16 * j + li;
            if (c >= d) continue;
            const T hc = h[b * d + c];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int64_t row = base + 16 * wave + M::row(lk, r);
                if (row < row_end) {
                    T v = acc[rc][j][r];
                    if constexpr (DIRECT) v += row == 0 ? -hc : (row == L ? hc : T(0));
                    else v += hc;
                    o[row * d + c] = v;
                }
            }
        }
    }
}

}  // namespace sigamd
