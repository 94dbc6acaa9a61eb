// Kernels of the signature hot path: increment pre-pass, tree forward sweep,
// tree reverse sweep, increment-gradient fold-back and the closed-form cases.
#pragma once
#include "sig_tree.h"

namespace sigamd {

template <int V>
struct IntC { static constexpr int value = V; };

// calls f(IntC<E>{}) for E = LO .. HI with E usable as a constant expression
template <int LO, int HI, typename F>
__device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (LO <= HI) {
        f(IntC<LO>{});
        static_for<LO + 1, HI>(f);
    }
}

// ---------------------------------------------------------------------------
// Increment pre-pass: z[b][t][c] of the (virtually) augmented path.
// lead-lag: even step moves the lead half, odd step the lag half; time is the
// last channel with constant spacing end_time / (len_eff - 1)
// (siglib/cpsig/cp_path.h:46-62,262-279; siglib/cusig/cu_signature.cu:146-166).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void increments_kernel(
    const T* __restrict__ path, T* __restrict__ inc, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, T time_step)
{
    // Layout [batch][L + 2][d]: row t + 1 holds the increment of step t; rows 0 and L + 1 are zero so
    // that the sweeps may prefetch one row past either end of a path without a bounds test.
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int64_t rows = L + 2;
    const int64_t total = batch * rows * d;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock) {
        const int c = int(e % d);
        const int64_t row = (e / d) % rows;
        const int64_t b = e / (int64_t(d) * rows);
        const T* x = path + b * len_raw * d_raw;
        T v;
        if (row == 0 || row == rows - 1) {
            v = T(0);
        } else {
            const int64_t t = row - 1;
            if (time_aug && c == d - 1) {
                v = T(t + 1) * time_step - T(t) * time_step;
            } else if (!lead_lag) {
                v = x[(t + 1) * d_raw + c] - x[t * d_raw + c];
            } else {
                const int64_t k = t >> 1;
                const bool odd = t & 1;
                if (c < d_raw) v = odd ? x[(k + 1) * d_raw + c] - x[k * d_raw + c] : T(0);
                else v = odd ? T(0) : x[(k + 1) * d_raw + (c - d_raw)] - x[k * d_raw + (c - d_raw)];
            }
        }
        inc[e] = v;
    }
}

// ---------------------------------------------------------------------------
// Lane set-up shared by both sweeps.
// ---------------------------------------------------------------------------
template <typename T, int D, int N, int TAIL, int K>
struct LaneCtx {
    using Tr = Tree<T, D, N, TAIL, K>;
    static constexpr int M = Tr::M;
    static constexpr bool WIDE = D > 0 && ipow64(D > 0 ? D : 1, M) >= 48;
    int d;
    TreeGeom G;
    LaneId id;
    int p[M];
    int a0;

    __device__ __forceinline__ void init(int d_rt, int64_t batch)
    {
        d = D > 0 ? D : d_rt;
        G = make_geom(d, M, K, D > 0);
        id = lane_id<WIDE>(G, batch);
        // idle lanes shadow a valid lane so that every load stays in bounds;
        // they never store and never contribute
        if constexpr (WIDE) {
            // path and group stay wave-uniform (waves past the batch exit before loading)
            if (id.q >= G.P) id.q = G.P - 1;
        } else if (!id.active) {
            if (id.b >= batch) id.b = batch - 1;
            if (id.q >= G.P) id.q = G.P - 1;
            if (id.g >= G.ng) id.g = G.ng - 1;
        }
        int64_t q = id.q;
#pragma unroll
        for (int l = M - 1; l >= 0; --l) {
            p[l] = int(q % d);
            q /= d;
        }
        a0 = id.g * K;
    }

    __device__ __forceinline__ void load_inc(typename Tr::Inc& in, const T* __restrict__ row) const
    {
        if constexpr (TAIL >= 2) {
#pragma unroll
            for (int j = 0; j < Tr::DD; ++j) in.z[j] = row[j];
        }
#pragma unroll
        for (int a = 0; a < K; ++a) in.zs[a] = (a0 + a < d) ? row[a0 + a] : T(0);
#pragma unroll
        for (int l = 0; l < M; ++l) in.pz[l] = row[p[l]];
    }

    // offset of level `lev` (1-based) inside a signature row
    __device__ __forceinline__ int64_t level_off(int lev, int scalar) const
    {
        int64_t o = scalar ? 1 : 0, sz = d;
        for (int i = 1; i < lev; ++i) { o += sz; sz *= d; }
        return o;
    }
};

// Nothing may be scheduled across this point: the loads above it are issued
// before any of the arithmetic below it.
__device__ __forceinline__ void loads_issued()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// all outstanding vector- and scalar-memory loads have landed
__device__ __forceinline__ void wait_all_loads()
{
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0);
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

template <typename T, int D, int N, int TAIL, int K>
__device__ __forceinline__ typename Tree<T, D, N, TAIL, K>::Inc negate(const typename Tree<T, D, N, TAIL, K>::Inc& in)
{
    using Tr = Tree<T, D, N, TAIL, K>;
    typename Tr::Inc o;
#pragma unroll
    for (int j = 0; j < Tr::DD; ++j) o.z[j] = -in.z[j];
#pragma unroll
    for (int a = 0; a < K; ++a) o.zs[a] = -in.zs[a];
#pragma unroll
    for (int l = 0; l < Tr::M; ++l) o.pz[l] = -in.pz[l];
    return o;
}

// ---------------------------------------------------------------------------
// Forward sweep.
// ---------------------------------------------------------------------------
template <typename T, int D, int N, int TAIL, int K>
__global__ __launch_bounds__(kBlock) void tree_fwd_kernel(
    const T* __restrict__ inc, T* __restrict__ out, int64_t batch, int64_t L, int d_rt,
    int64_t out_stride, int scalar, int nseg, int64_t lseg)
{
    // `batch` counts (path, time segment) pairs: item vb = path * nseg + segment sweeps the
    // increments [segment * lseg, min(L, (segment + 1) * lseg)) and stores the signature of
    // that piece in row vb of `out`.  nseg == 1 is the plain whole-path sweep.
    using Tr = Tree<T, D, N, TAIL, K>;
    constexpr int M = Tr::M;
    LaneCtx<T, D, N, TAIL, K> cx;
    cx.init(d_rt, batch);
    if constexpr (LaneCtx<T, D, N, TAIL, K>::WIDE) {
        if (cx.id.b >= batch) return;   // uniform: the whole wave is past the batch
    }
    const int d = cx.d;

    Tr S;
#pragma unroll
    for (int l = 0; l < M; ++l) S.c[l] = T(0);
#pragma unroll
    for (int i = 0; i < Tr::SUB; ++i) S.s[i] = T(0);

    // Two increment buffers used alternately: the loads of step t+1 are issued
    // before the arithmetic of step t and waited for after it, so neither the
    // scalar-cache nor the vector-memory latency sits on the critical path.
    const int64_t seg = cx.id.b % nseg;
    const int64_t t0 = seg * lseg;
    const int64_t ns = (L - t0 < lseg) ? L - t0 : lseg;      // steps of this segment (>= 1)
    const T* row = inc + ((cx.id.b / nseg) * (L + 2) + 1 + t0) * d;     // row of the segment's first step
    typename Tr::Inc za, zb;
    cx.load_inc(za, row);
    wait_all_loads();
    int64_t t = 0;
    for (; t + 2 <= ns; t += 2) {
        cx.load_inc(zb, row + d);
        loads_issued();
        S.fwd_step(za);
        wait_all_loads();
        cx.load_inc(za, row + 2 * d);          // at most one row past the path: the zero guard row
        loads_issued();
        S.fwd_step(zb);
        wait_all_loads();
        row += 2 * d;
    }
    if (t < ns) S.fwd_step(za);

    if (!cx.id.active) return;
    T* o = out + cx.id.b * out_stride;
    if (scalar && cx.id.q == 0 && cx.id.g == 0) o[0] = T(1);
    // chain nodes are stored by the lane whose remaining prefix letters are 0
    {
        int64_t rest = 1;   // d^(M-l)
#pragma unroll
        for (int l = M; l >= 1; --l) {
            if (cx.id.g == 0 && cx.id.q % rest == 0) o[cx.level_off(l, scalar) + cx.id.q / rest] = S.c[l - 1];
            rest *= d;
        }
    }
    static_for<1, TAIL>([&](auto ec) {
        constexpr int e = decltype(ec)::value;
        constexpr int sub = int(ipow64(Tr::DD, e - 1));   // values below one depth-1 letter
        const int64_t lo = cx.level_off(M + e, scalar);
#pragma unroll
        for (int a = 0; a < K; ++a) {
            if (cx.a0 + a < d) {
                const int64_t base = lo + (cx.id.q * d + cx.a0 + a) * sub;
#pragma unroll
                for (int r = 0; r < sub; ++r) o[base + r] = S.s[Tr::off(e) + a * sub + r];
            }
        }
    });
}

// ---------------------------------------------------------------------------
// Reverse sweep: per step un-multiply the state by exp(-z), pull the adjoint
// back through the step, emit the increment gradient.
// (siglib/cpsig/cp_signature.h:1137-1187)
// ---------------------------------------------------------------------------
// LDS tile of the wide-layout reduction: one row per (step-in-chunk, letter), two
// half-rows of 32 lanes padded to 33 so that writers and the summing lanes both
// hit distinct banks.
constexpr int kRedStride = 66;
__host__ __device__ constexpr int bwd_chunk(int d) { return (31 / d) < 1 ? 1 : ((31 / d) > 8 ? 8 : (31 / d)); }

template <typename T>
__device__ __forceinline__ void lds_add(T* p, T v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
template <typename T>
__device__ __forceinline__ void dev_add(T* p, T v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename T, int D, int N, int TAIL, int K>
__global__ __launch_bounds__(kBlock) void tree_bwd_kernel(
    const T* __restrict__ inc, const T* __restrict__ sig, const T* __restrict__ gsig,
    T* __restrict__ dzinc, int64_t batch, int64_t L, int d_rt, int64_t sig_stride, int scalar,
    int use_lds)
{
    using Tr = Tree<T, D, N, TAIL, K>;
    using Ad = TreeAdj<T, D, N, TAIL, K>;
    using Cx = LaneCtx<T, D, N, TAIL, K>;
    constexpr int M = Tr::M;
    extern __shared__ double lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);

    Cx cx;
    cx.init(d_rt, batch);
    if constexpr (Cx::WIDE) {
        if (cx.id.b >= batch) return;
    }
    const int d = cx.d;
    const bool active = cx.id.active;

    // ---- load state and upstream gradient -------------------------------
    Tr S;
    Ad A;
    const T* srow = sig + cx.id.b * sig_stride;
    const T* grow = gsig + cx.id.b * sig_stride;
    {
        int64_t rest = 1;
#pragma unroll
        for (int l = M; l >= 1; --l) {
            const int64_t idx = cx.level_off(l, scalar) + cx.id.q / rest;
            S.c[l - 1] = srow[idx];
            const bool owner = active && cx.id.g == 0 && cx.id.q % rest == 0;
            A.gc[l - 1] = owner ? grow[idx] : T(0);
            rest *= d;
        }
    }
    static_for<1, TAIL>([&](auto ec) {
        constexpr int e = decltype(ec)::value;
        constexpr int sub = int(ipow64(Tr::DD, e - 1));
        const int64_t lo = cx.level_off(M + e, scalar);
#pragma unroll
        for (int a = 0; a < K; ++a) {
            const bool ok = cx.a0 + a < d;
            const int64_t base = lo + (cx.id.q * d + (ok ? cx.a0 + a : 0)) * sub;
#pragma unroll
            for (int r = 0; r < sub; ++r) {
                S.s[Tr::off(e) + a * sub + r] = ok ? srow[base + r] : T(0);
                A.gs[Tr::off(e) + a * sub + r] = (ok && active) ? grow[base + r] : T(0);
            }
        }
    });

    // ---- reduction of the per-lane increment-gradient pieces ------------
    // wide layout: every lane writes its D partial sums of a step into a
    // [row = step-in-chunk * D + letter][lane] tile in LDS (chain pieces are added
    // into the lane's own column); once the chunk is full each row is summed by
    // a pair of lanes and added to dz[b][t][letter] in HBM.  packed layout:
    // per-wave accumulator [path-in-wave][letter] updated with LDS atomics.
    const int lane = threadIdx.x & (kWave - 1);
    const int wave_in_block = threadIdx.x >> 6;
    constexpr bool WIDE = Cx::WIDE;
    constexpr int CH = bwd_chunk(Tr::DD);
    const int slots = cx.G.ppw;
    T* wbuf;
    if constexpr (WIDE) wbuf = lds + wave_in_block * (CH * Tr::DD * kRedStride);
    else wbuf = lds + int64_t(wave_in_block) * slots * d;
    T* acc = wbuf + int64_t(cx.id.slot) * d;
    const int woff = (lane >> 5) * 33 + (lane & 31);
    if constexpr (!WIDE) {
        if (use_lds) {
            for (int e = lane; e < slots * d; e += kWave) wbuf[e] = T(0);
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
            __builtin_amdgcn_wave_barrier();
        }
    }
    int64_t b_first;
    {
        const int64_t wave = int64_t(blockIdx.x) * kWavesPerBlock + wave_in_block;
        b_first = (cx.G.ppw > 1) ? wave * cx.G.ppw : (wave / cx.G.wpp);
    }
    int cs = 0;                 // rows of the current chunk already filled (in steps)
    int64_t t_chunk = L - 1;    // step held by chunk slot 0

    auto reduce_chunk = [&](int n_slots) {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        const int n_rows = n_slots * Tr::DD;
        for (int h = lane; h < 2 * n_rows; h += kWave) {
            const int rowi = h >> 1, half = h & 1;
            const T* src = wbuf + rowi * kRedStride + half * 33;
            T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
#pragma unroll
            for (int i = 0; i < 32; i += 4) {
                s0 += src[i];
                s1 += src[i + 1];
                s2 += src[i + 2];
                s3 += src[i + 3];
            }
            T sum = (s0 + s1) + (s2 + s3);
            sum += __shfl_xor(sum, 1);
            if (half == 0) {
                const int slot = rowi / Tr::DD, j = rowi % Tr::DD;
                dev_add(&dzinc[(cx.id.b * L + (t_chunk - slot)) * d + j], sum);
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
        __builtin_amdgcn_wave_barrier();
    };

    auto do_step = [&](const typename Tr::Inc& z, int64_t t) {
        S.fwd_step(negate<T, D, N, TAIL, K>(z));     // state before the step
        typename Ad::DInc dz;
#pragma unroll
        for (int j = 0; j < Tr::DD; ++j) dz.dj[j] = T(0);
#pragma unroll
        for (int a = 0; a < K; ++a) dz.da[a] = T(0);
#pragma unroll
        for (int l = 0; l < M; ++l) dz.dc[l] = T(0);
        A.pullback(S, z, dz);

        if constexpr (WIDE) {
            T* tile = wbuf + cs * (Tr::DD * kRedStride) + woff;
#pragma unroll
            for (int j = 0; j < Tr::DD; ++j) tile[j * kRedStride] = (active && TAIL >= 2) ? dz.dj[j] : T(0);
            if (active) {
                // depth-1 letters (wave-uniform rows) and chain letters (per-lane rows) are
                // added into the lane's own column; LDS executes a wave's operations in order
#pragma unroll
                for (int a = 0; a < K; ++a)
                    if (cx.a0 + a < Tr::DD) lds_add(&tile[(cx.a0 + a) * kRedStride], dz.da[a]);
#pragma unroll
                for (int l = 0; l < M; ++l) lds_add(&tile[cx.p[l] * kRedStride], dz.dc[l]);
            }
            ++cs;
            if (cs == CH || t == 0) {
                reduce_chunk(cs);
                cs = 0;
                t_chunk = t - 1;
            }
        } else {
            T* grow_t = dzinc + (cx.id.b * L + t) * d;
            if (use_lds) {
                if (active) {
#pragma unroll
                    for (int a = 0; a < K; ++a)
                        if (cx.a0 + a < d) lds_add(&acc[cx.a0 + a], dz.da[a]);
                    if constexpr (TAIL >= 2) {
#pragma unroll
                        for (int j = 0; j < Tr::DD; ++j) lds_add(&acc[j], dz.dj[j]);
                    }
#pragma unroll
                    for (int l = 0; l < M; ++l) lds_add(&acc[cx.p[l]], dz.dc[l]);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                for (int e = lane; e < slots * d; e += kWave) {
                    const T v = wbuf[e];
                    wbuf[e] = T(0);
                    const int64_t bb = b_first + e / d;
                    if (bb < batch) dev_add(&dzinc[(bb * L + t) * d + e % d], v);
                }
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                __builtin_amdgcn_wave_barrier();
            } else if (active) {
                if constexpr (TAIL >= 2) {
#pragma unroll
                    for (int j = 0; j < Tr::DD; ++j) dev_add(&grow_t[j], dz.dj[j]);
                }
#pragma unroll
                for (int a = 0; a < K; ++a)
                    if (cx.a0 + a < d) dev_add(&grow_t[cx.a0 + a], dz.da[a]);
#pragma unroll
                for (int l = 0; l < M; ++l) dev_add(&grow_t[cx.p[l]], dz.dc[l]);
            }
        }
    };

    // reverse sweep with two alternating increment buffers (see the forward kernel)
    const T* row = inc + (cx.id.b * (L + 2) + L) * d;      // row of the last step
    typename Tr::Inc za, zb;
    cx.load_inc(za, row);
    wait_all_loads();
    int64_t t = L - 1;
    for (; t >= 1; t -= 2) {
        cx.load_inc(zb, row - d);
        loads_issued();
        do_step(za, t);
        wait_all_loads();
        cx.load_inc(za, row - 2 * d);          // at most the zero guard row in front of the path
        loads_issued();
        do_step(zb, t - 1);
        wait_all_loads();
        row -= 2 * d;
    }
    if (t == 0) do_step(za, 0);
}

// ---------------------------------------------------------------------------
// Increment gradient -> raw path gradient.  Point i of the raw path receives
// +dz of every step that ends in it and -dz of every step that starts from it;
// with lead-lag, step 2k moves the lead half and step 2k+1 the lag half of
// raw segment k -> k+1; the time channel has no raw counterpart
// (siglib/cpsig/cp_signature.h:1189-1201, siglib/cusig/cu_path_transforms.cu:129-147).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void path_grad_kernel(
    const T* __restrict__ dzinc, T* __restrict__ out, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag)
{
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const int64_t total = batch * len_raw * d_raw;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock) {
        const int c = int(e % d_raw);
        const int64_t i = (e / d_raw) % len_raw;
        const int64_t b = e / (int64_t(d_raw) * len_raw);
        const T* g = dzinc + b * L * d;
        T v = T(0);
        if (!lead_lag) {
            if (i > 0) v += g[(i - 1) * d + c];
            if (i < len_raw - 1) v -= g[i * d + c];
        } else {
            if (i > 0) v += g[(2 * (i - 1)) * d + d_raw + c] + g[(2 * (i - 1) + 1) * d + c];
            if (i < len_raw - 1) v -= g[(2 * i) * d + d_raw + c] + g[(2 * i + 1) * d + c];
        }
        out[e] = v;
    }
}

// ---------------------------------------------------------------------------
// Closed forms (siglib/cpsig/cp_signature.h:748-784,845-851; backward :941-945).
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_trivial_kernel(T* __restrict__ out, int64_t batch, int64_t stride, int scalar)
{
    const int64_t total = batch * stride;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock)
        out[e] = (scalar && e % stride == 0) ? T(1) : T(0);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void zero_kernel(T* __restrict__ out, int64_t total)
{
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock)
        out[e] = T(0);
}

// degree 1: endpoint difference of the augmented path
template <typename T>
__global__ __launch_bounds__(kBlock) void degree_one_fwd_kernel(
    const T* __restrict__ path, T* __restrict__ out, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, T time_step, int scalar)
{
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t len = lead_lag ? 2 * len_raw - 1 : len_raw;
    const int64_t stride = d + (scalar ? 1 : 0);
    const int64_t total = batch * stride;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock) {
        const int64_t b = e / stride;
        int c = int(e % stride);
        if (scalar) {
            if (c == 0) { out[e] = T(1); continue; }
            --c;
        }
        const T* x = path + b * len_raw * d_raw;
        T v;
        if (time_aug && c == d - 1) v = T(len) * time_step - time_step;
        else {
            const int cr = c < d_raw ? c : c - d_raw;
            v = x[(len_raw - 1) * d_raw + cr] - x[cr];
        }
        out[e] = v;
    }
}

// effective dimension 1: level k = Delta^k / k!
template <typename T>
__global__ __launch_bounds__(kBlock) void dim_one_fwd_kernel(
    const T* __restrict__ path, T* __restrict__ out, int64_t batch, int64_t len_raw, int degree, int scalar)
{
    for (int64_t b = int64_t(blockIdx.x) * kBlock + threadIdx.x; b < batch; b += int64_t(gridDim.x) * kBlock) {
        const T inc = path[b * len_raw + len_raw - 1] - path[b * len_raw];
        T* o = out + b * (degree + (scalar ? 1 : 0));
        T v = T(1);
        if (scalar) *o++ = v;
        for (int k = 1; k <= degree; ++k) {
            v *= inc / T(k);
            *o++ = v;
        }
    }
}

// degree 1 backward: every step's increment gradient equals the level-1
// upstream gradient, so only the two endpoints of the raw path receive it.
template <typename T>
__global__ __launch_bounds__(kBlock) void degree_one_bwd_kernel(
    const T* __restrict__ gsig, T* __restrict__ out, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, int scalar)
{
    const int d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t stride = d + (scalar ? 1 : 0);
    const int64_t total = batch * len_raw * d_raw;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock) {
        const int c = int(e % d_raw);
        const int64_t i = (e / d_raw) % len_raw;
        const int64_t b = e / (int64_t(d_raw) * len_raw);
        const T* g = gsig + b * stride + (scalar ? 1 : 0);
        T v = g[c];
        if (lead_lag) v += g[d_raw + c];
        T r = T(0);
        if (i == len_raw - 1) r += v;
        if (i == 0) r -= v;
        out[e] = r;
    }
}

// ---------------------------------------------------------------------------
// Chen product C = A (x) B of two signatures per path (scalar terms implicit 1):
//   C_t[w] = A_t[w] + B_t[w] + sum_{k=1..t-1} A_k[w_1..w_k] * B_{t-k}[w_{k+1}..w_t]
// (siglib/cpsig/cp_sig_combine.h:35-66).  One thread per output coefficient; rows
// of A, B, C may have different strides and C may carry a leading scalar slot.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kBlock) void sig_combine_kernel(
    const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int64_t batch, int d, int degree,
    int64_t sig_len /* sum_{k=1..degree} d^k */, int64_t a_stride, int64_t b_stride, int64_t c_stride,
    int a_off, int b_off, int c_off)
{
    const int64_t total = batch * sig_len;
    for (int64_t e = int64_t(blockIdx.x) * kBlock + threadIdx.x; e < total; e += int64_t(gridDim.x) * kBlock) {
        const int64_t b = e / sig_len;
        int64_t r = e % sig_len;
        // level t and word index w of coefficient r
        int t = 1;
        int64_t lvl = d, lo = 0;
        while (r >= lo + lvl) { lo += lvl; lvl *= d; ++t; }
        const int64_t w = r - lo;
        const T* a = A + b * a_stride + a_off;
        const T* bb = B + b * b_stride + b_off;
        T acc = a[lo + w] + bb[lo + w];
        // split w after its first k letters: prefix index w / d^(t-k), suffix index w % d^(t-k)
        int64_t div = lvl / d;          // d^(t-1)
        int64_t a_lo = 0, a_sz = d;     // level k of A
        int64_t b_lo = lo - div;        // start of level t-1 of B
        int64_t b_sz = div;
        for (int k = 1; k < t; ++k) {
            acc = fmadd(a[a_lo + w / div], bb[b_lo + w % div], acc);
            a_lo += a_sz; a_sz *= d;
            b_sz /= d; b_lo -= b_sz;
            div /= d;
        }
        T* c = C + b * c_stride;
        c[c_off + r] = acc;
        if (c_off && r == 0) c[0] = T(1);
    }
}

}  // namespace sigamd
