// Kernels of the signature hot path: increment pre-pass, tree forward sweep,
// tree reverse sweep, increment-gradient fold-back and the closed-form cases.
#pragma once
#include <atomic>
#include <limits>

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
// Lane set-up shared by both sweeps.
// ---------------------------------------------------------------------------
template <typename T, int D, int N, int TAIL, int K>
struct LaneCtx {
    using Tr = Tree<T, D, N, TAIL, K>;
    static constexpr int M = Tr::M;
    static constexpr bool WIDE = D > 0 ? ipow64(D > 0 ? D : 1, M) >= 48 : D < 0;
    static constexpr bool kWholeGroups = D > 0 && D % K == 0;     // no letter group reaches past the row
    static constexpr bool kRunTimeWide = D < 0;
    int d;
    TreeGeom G;
    LaneId id;
    int p[M];
    int a0;

    __device__ __forceinline__ void init(int d_rt, int64_t batch, bool xcd = true)
    {
        d = D > 0 ? D : d_rt;
        G = make_geom(d, M, K, D != 0);
        id = lane_id<WIDE>(G, batch, xcd);
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
        a0 = kRunTimeWide ? __builtin_amdgcn_readfirstlane(id.g * K) : id.g * K;      // wave-uniform: say so
    }

    // GUARD: every read of the group is bounds-tested instead (no read past the row, no merged loads)
    template <bool GUARD = false>
    __device__ __forceinline__ void load_inc(typename Tr::Inc& in, const T* __restrict__ row) const
    {
        if constexpr (TAIL >= 2) {
#pragma unroll
            for (int j = 0; j < Tr::DD; ++j) in.z[j] = row[j];
        }
        // Run-time dimension, wide layout: the group is wave-uniform and its K reads merge into a few wide scalar loads,
        // provided none of them is guarded.  The last group of a row then reads on into the next row (the increment
        // buffer continues for more than K elements past its last row) and mask_inc drops what lies beyond the row.
        if constexpr (kWholeGroups || (D < 0 && !GUARD)) {
#pragma unroll
            for (int a = 0; a < K; ++a) in.zs[a] = row[a0 + a];
        } else {
#pragma unroll
            for (int a = 0; a < K; ++a) in.zs[a] = (a0 + a < d) ? row[a0 + a] : T(0);
        }
#pragma unroll
        for (int l = 0; l < M; ++l) in.pz[l] = row[p[l]];
    }

    // Zeroes the letters that load_inc read past the end of the row; needed by the waves of a row's last group when the
    // dimension is not a multiple of K (partial_group()).
    __device__ __forceinline__ void mask_inc(typename Tr::Inc& in) const
    {
#pragma unroll
        for (int a = 0; a < K; ++a) in.zs[a] = (a0 + a < d) ? in.zs[a] : T(0);
    }
    __device__ __forceinline__ bool partial_group() const { return D < 0 && a0 + K > d; }      // wave-uniform

    // offset of level `lev` (1-based) inside a signature row
    __device__ __forceinline__ int64_t level_off(int lev, int scalar) const
    {
        int64_t o = scalar ? 1 : 0, sz = d;
        for (int i = 1; i < lev; ++i) { o += sz; sz *= d; }
        return o;
    }
};

// NaN or infinity
__device__ __forceinline__ bool not_finite(double v) { return !(__builtin_fabs(v) <= std::numeric_limits<double>::max()); }
__device__ __forceinline__ bool not_finite(float v) { return !(__builtin_fabsf(v) <= std::numeric_limits<float>::max()); }

// product rounded on its own: the empty asm hides it from the compiler, which would otherwise contract it into a
// multiply-add with a neighbouring operation
template <typename T>
__device__ __forceinline__ T mul_rn(T a, T b)
{
    T p = a * b;
    asm volatile("" : "+v"(p));
    return p;
}

// Nothing may be scheduled across this point: the loads above it are issued
// before any of the arithmetic below it.
__device__ __forceinline__ void loads_issued()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

// All LDS operations of this wave have completed (vector-memory counters untouched).  Placed before the ring reads
// of the next step it replaces the compiler's waits before every first use of the current step's values (read a
// whole step ago): a wait that does not stall still takes one of a lone wave's issue slots.
__device__ __forceinline__ void wait_lds()
{
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0xc07f);     // lgkmcnt(0), vmcnt and expcnt at their maxima
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


// ---------------------------------------------------------------------------
// Sweep drivers: feed the increments of steps first, first + DIR, ... (count
// steps) to step(z, t).  Two ways of getting an increment row to a wave:
//
//  * scalar path (any layout): the row is read where it lies in HBM/L2 with two
//    alternating register sets; the loads of the next step are issued before the
//    arithmetic of the current one.  In the wide layout the row address is
//    wave-uniform, so the row arrives in SGPRs through the scalar cache.
//
//  * staged path (wide layout only): every wave copies chunks of kStageSteps
//    rows into a private LDS ring two chunks ahead of use (ordinary vector loads,
//    so HBM latency is hidden by a whole chunk of arithmetic) and reads each row
//    back with broadcast LDS reads one step ahead.  The row then sits in VGPRs:
//    an FMA whose operands are all VGPRs issues faster than one reading an SGPR
//    when a SIMD holds only one or two waves, which is the regime of small batches.
// ---------------------------------------------------------------------------
constexpr int kStageSteps = 16;

template <typename T, int D, int DIR>
struct IncRing {
    static constexpr int CS = kStageSteps;
    static constexpr int CHUNK = CS * D;                       // elements per chunk
    static constexpr int NREG = (CHUNK + kWave - 1) / kWave;   // elements per lane per chunk
    static constexpr int ELEMS = 2 * CHUNK + D;                // two chunks and one wrap row
    // DIR > 0: [even chunk][odd chunk][copy of row 0 of the even chunk]
    // DIR < 0: [copy of the last row of the even chunk][odd chunk][even chunk]
    __host__ __device__ static constexpr int base(int parity)
    {
        return DIR > 0 ? parity * CHUNK : D + (1 - parity) * CHUNK;
    }
    // The ring can also be fed from the points of a plain path (no augmentation): element e of a chunk is then
    // x[e + D] - x[e], the two loads travel in `regs` and `ahead` and are subtracted when the chunk is committed.
    // Only narrow paths get the second register set.
    static constexpr bool kPoints = NREG <= 4;
    T* lds;
    int lane;
    T regs[NREG];
    T ahead[kPoints ? NREG : 1];

    __device__ __forceinline__ void issue(const T* __restrict__ g)
    {
#pragma unroll
        for (int i = 0; i < NREG; ++i) {
            const int e = lane + kWave * i;
            regs[i] = ((i + 1) * kWave <= CHUNK || e < CHUNK) ? g[e] : T(0);
        }
    }
    // g: the point whose increment is element 0 of the chunk; elements outside [lo, hi) are not read and count as 0
    // (nothing before the first or after the last point of the swept range is touched)
    __device__ __forceinline__ void issue_points(const T* __restrict__ g, int lo, int hi)
    {
        if constexpr (kPoints) {
#pragma unroll
            for (int i = 0; i < NREG; ++i) {
                const int e = lane + kWave * i;
                const bool ok = e >= lo && e < hi;
                regs[i] = ok ? g[e] : T(0);
                ahead[i] = ok ? g[e + D] : T(0);
            }
        }
    }
    __device__ __forceinline__ void commit(int parity, bool points = false)
    {
        T* dst = lds + base(parity);
#pragma unroll
        for (int i = 0; i < NREG; ++i) {
            const int e = lane + kWave * i;
            if ((i + 1) * kWave <= CHUNK || e < CHUNK) {
                T v = regs[i];
                if constexpr (kPoints) {
                    if (points) v = ahead[i] - v;
                }
                dst[e] = v;
                if (parity == 0) {
                    if (DIR > 0) { if (e < D) lds[2 * CHUNK + e] = v; }
                    else { if (e >= CHUNK - D) lds[e - (CHUNK - D)] = v; }
                }
            }
        }
    }
};

template <typename T>
__device__ __forceinline__ const T* opaque_lds(const T* p)
{
    typedef const T __attribute__((address_space(3))) * LdsPtr;
    uint32_t a = uint32_t(reinterpret_cast<uintptr_t>((LdsPtr)p));
    asm volatile("" : "+v"(a));
    return (const T*)reinterpret_cast<LdsPtr>(uintptr_t(a));
}

// scalar path.  WAIT_ALL: end every step with a full wait for outstanding loads (cheapest schedule when the
// step issues no stores); the backward must not do that, because a full wait would also wait for the
// acknowledgement of the global atomics it fires, so there the compiler's per-register waits are used.
template <int DIR, bool WAIT_ALL, bool MASK, typename Cx, typename Inc, typename T, typename StepFn>
__device__ __forceinline__ void sweep_direct_rows(const Cx& cx, const T* __restrict__ row, int64_t first, int64_t count,
                                                  StepFn&& step)
{
    // MASK: the wave's letter group reaches past the row.  The forward reads it whole and zeroes the excess when the
    // row is used; the backward, short of registers, keeps bounds-tested reads there.
    constexpr bool GUARD = MASK && !WAIT_ALL;
    constexpr bool ZERO = MASK && !GUARD;
    // Scalar loads return out of order, so the only wait there is for them is "all landed".  The row a step uses was
    // requested a whole step ago: waiting for it before the next row is requested costs nothing, while any later first
    // use would also wait for the row just requested.  (The forward's full wait at the end of a step does the same.)
    constexpr bool ROW_WAIT = Cx::kRunTimeWide && !GUARD && !WAIT_ALL;
    const int d = cx.d;
    Inc za, zb;
    cx.template load_inc<GUARD>(za, row);
    if constexpr (Cx::kRunTimeWide && WAIT_ALL) wait_all_loads();
    int64_t i = 0;
    for (; i + 2 <= count; i += 2) {
        if constexpr (ROW_WAIT) wait_lds();
        cx.template load_inc<GUARD>(zb, row + DIR * d);
        loads_issued();
        if constexpr (ZERO) cx.mask_inc(za);
        step(za, first + DIR * i, IntC<-1>{}, IntC<0>{});
        if constexpr (WAIT_ALL) wait_all_loads();
        if constexpr (ROW_WAIT) wait_lds();
        cx.template load_inc<GUARD>(za, row + 2 * DIR * d);        // at most one row past the path: a zero guard row
        loads_issued();
        if constexpr (ZERO) cx.mask_inc(zb);
        step(zb, first + DIR * (i + 1), IntC<-1>{}, IntC<1>{});
        if constexpr (WAIT_ALL) wait_all_loads();
        row += 2 * DIR * d;
    }
    if (i < count) {
        if constexpr (ZERO) cx.mask_inc(za);
        step(za, first + DIR * i, IntC<-1>{}, IntC<0>{});
    }
}

// run-time-dimension wide kernels hold the loop twice, and each wave takes the one its letter group needs
template <int DIR, bool WAIT_ALL, typename Cx, typename Inc, typename T, typename StepFn>
__device__ __forceinline__ void sweep_direct(const Cx& cx, const T* __restrict__ row, int64_t first, int64_t count,
                                             StepFn&& step)
{
    if (Cx::kRunTimeWide && cx.partial_group()) sweep_direct_rows<DIR, WAIT_ALL, true, Cx, Inc>(cx, row, first, count, step);
    else sweep_direct_rows<DIR, WAIT_ALL, false, Cx, Inc>(cx, row, first, count, step);
}

// staged path; G0 >= 0: the depth-1 letters start at the compile-time letter G0
// points (wave-uniform; plain paths only): `row` is the path point at which the first step of the sweep starts, instead
// of that step's increment row, and the ring takes differences of consecutive points.
// step(increments, step index, IntC<G0>, IntC<position>): position 0 / 1 alternate from the first step of the range on
// (chunks hold an even number of steps), so a range that starts on an even step hands the step's parity to `step`
// as a compile-time constant.
template <int DIR, int G0, typename Tr, typename Cx, typename T, typename StepFn>
__device__ __forceinline__ void sweep_staged(const Cx& cx, const T* __restrict__ row, int64_t first, int64_t count,
                                             T* lds_wave, StepFn&& step, bool points = false)
{
    constexpr int D = Tr::DD;
    using Ring = IncRing<T, D, DIR>;
    constexpr int CS = Ring::CS;
    Ring ring;
    ring.lds = lds_wave;
    ring.lane = threadIdx.x & (kWave - 1);
    // memory start of chunk k: DIR > 0: row + k * CHUNK;  DIR < 0: the CS rows ending with the row of step first - k*CS
    auto chunk_src = [&](int64_t k) -> const T* {
        return DIR > 0 ? row + k * Ring::CHUNK : row - (k * CS + (CS - 1)) * D;
    };
    const int64_t nchunks = (count + CS - 1) / CS;

    auto load_row = [&](typename Tr::Inc& in, const T* lp) {
        if constexpr (Tr::TAIL_ >= 2) {
#pragma unroll
            for (int j = 0; j < D; ++j) in.z[j] = lp[j];
        }
#pragma unroll
        for (int a = 0; a < Tr::K_; ++a) {
            if constexpr (G0 >= 0 && Tr::TAIL_ >= 2) in.zs[a] = (G0 + a < D) ? in.z[(G0 + a < D) ? G0 + a : 0] : T(0);
            else if constexpr (G0 >= 0) in.zs[a] = (G0 + a < D) ? lp[(G0 + a < D) ? G0 + a : 0] : T(0);
            else in.zs[a] = (cx.a0 + a < D) ? lp[cx.a0 + a] : T(0);
        }
#pragma unroll
        for (int l = 0; l < Tr::M; ++l) in.pz[l] = lp[cx.p[l]];
    };

    // chunk k holds the elements [k * CHUNK, (k + 1) * CHUNK) of the range; count * D of them exist
    auto issue = [&](int64_t k) {
        if (Ring::kPoints && points) {
            if (DIR > 0) {
                const int64_t left = count * D - k * Ring::CHUNK;
                ring.issue_points(chunk_src(k), 0, left < Ring::CHUNK ? int(left) : Ring::CHUNK);
            } else {
                // the chunk ends with the row of local step count - 1 - k * CS; rows of steps before the range are not read
                const int64_t before = (k + 1) * CS - count;
                ring.issue_points(chunk_src(k), before > 0 ? int(before) * D : 0, Ring::CHUNK);
            }
        } else {
            ring.issue(chunk_src(k));
        }
    };
    issue(0);
    ring.commit(0, points);
    if (nchunks > 1) issue(1);
    typename Tr::Inc za, zb;
    load_row(za, ring.lds + Ring::base(0) + (DIR > 0 ? 0 : (CS - 1) * D));
    int64_t done = 0;
    for (int64_t k = 0; k < nchunks; ++k) {
        const int parity = int(k & 1);
        if (k + 1 < nchunks) ring.commit(parity ^ 1, points);    // chunk k+1 becomes readable
        if (k + 2 < nchunks) issue(k + 2);                       // two chunks ahead of use
        // the row pointer is made opaque so that row reads use small immediate offsets from one VGPR
        const T* lp = opaque_lds(ring.lds + Ring::base(parity) + (DIR > 0 ? 0 : (CS - 1) * D));
        const int nk = int((count - done < CS) ? count - done : CS);
        int i = 0;
        for (; i + 2 <= nk; i += 2) {
            // forward only: the backward's steps end with LDS adds into the reduction tile, which such a wait would sit out
            if constexpr (DIR > 0) wait_lds();
            load_row(zb, lp + DIR * D);
            loads_issued();
            step(za, first + DIR * (done + i), IntC<G0>{}, IntC<0>{});
            if constexpr (DIR > 0) wait_lds();
            load_row(za, lp + 2 * DIR * D);                      // may be row 0 of the next chunk (contiguous or wrap copy)
            loads_issued();
            step(zb, first + DIR * (done + i + 1), IntC<G0>{}, IntC<1>{});
            lp += 2 * DIR * D;
        }
        if (i < nk) step(za, first + DIR * (done + i), IntC<G0>{}, IntC<0>{});          // odd tail: only in the last chunk
        done += nk;
    }
}

// ---------------------------------------------------------------------------
// Forward sweep.
// ---------------------------------------------------------------------------
// LL: the increments have lead-lag structure (1: with a time channel as last letter, D odd; 2: without, D even) and every
// range handed to a wave starts on an even step (lseg even): steps then skip the letters that cannot move (LeadLagLetters).
template <typename T, int D, int N, int TAIL, int K, bool ZL, int LL = 0>
__global__ __launch_bounds__(kBlock) void tree_fwd_kernel(
    const T* __restrict__ inc, T* __restrict__ out, int64_t batch, int64_t L, int d_rt,
    int64_t out_stride, int scalar, int nseg, int64_t lseg, int* __restrict__ nonfinite, int from_points)
{
    static_assert(LL == 0 || (ZL && D >= 2 && ((LL == 1) == ((D & 1) == 1))), "lead-lag variants: staged, time channel iff D is odd");
    // `nonfinite` (may be null): set to 1 when any stored value is NaN or infinite.
    // `from_points` (staged kernels of narrow paths only): `inc` is the plain path [batch][L + 1][d] itself and the
    // increments are formed while they are staged.
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

    const int64_t seg = cx.id.b % nseg;
    const int64_t t0 = seg * lseg;
    const int64_t ns = (L - t0 < lseg) ? L - t0 : lseg;      // steps of this segment (>= 1)
    // row of the segment's first step (increments: [batch][L + 2][d] with a zero row at either end)
    const T* row = from_points ? inc + ((cx.id.b / nseg) * (L + 1) + t0) * d : inc + ((cx.id.b / nseg) * (L + 2) + 1 + t0) * d;
    auto step = [&](const typename Tr::Inc& z, int64_t, auto g0c, auto pos) {
        if constexpr (LL == 0) S.fwd_step(z);
        else S.template fwd_step<LeadLagLetters<Tr::DD, decltype(pos)::value, decltype(g0c)::value>>(z);
    };
    if constexpr (ZL) {
        static_assert(LaneCtx<T, D, N, TAIL, K>::WIDE, "staged increments need the wide layout");
        extern __shared__ double lds_raw_f[];
        T* lds_wave = reinterpret_cast<T*>(lds_raw_f) + (threadIdx.x >> 6) * IncRing<T, Tr::DD, 1>::ELEMS;
        constexpr int NG = (Tr::DD + K - 1) / K;
        const bool points = IncRing<T, Tr::DD, 1>::kPoints && from_points != 0;
        if constexpr (NG <= 3) {
            static_for<0, NG - 1>([&](auto gc) {
                if (cx.id.g == decltype(gc)::value)
                    sweep_staged<1, decltype(gc)::value * K, Tr>(cx, row, t0, ns, lds_wave, step, points);
            });
        } else {
            sweep_staged<1, -1, Tr>(cx, row, t0, ns, lds_wave, step, points);
        }
    } else {
        sweep_direct<1, true, LaneCtx<T, D, N, TAIL, K>, typename Tr::Inc>(cx, row, t0, ns, step);
    }

    if (!cx.id.active) return;
    T* o = out + cx.id.b * out_stride;
    if (scalar && cx.id.q == 0 && cx.id.g == 0) o[0] = T(1);
    // chk stays 0 while every value is finite: x * 0 is NaN for x = NaN or +-Inf
    T chk = T(0);
    // chain nodes are stored by the lane whose remaining prefix letters are 0
    {
        int64_t rest = 1;   // d^(M-l)
#pragma unroll
        for (int l = M; l >= 1; --l) {
            if (cx.id.g == 0 && cx.id.q % rest == 0) o[cx.level_off(l, scalar) + cx.id.q / rest] = S.c[l - 1];
            chk = fmadd(S.c[l - 1], T(0), chk);
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
#pragma unroll
    for (int i = 0; i < Tr::SUB; ++i) chk = fmadd(S.s[i], T(0), chk);      // unused slots hold 0
    if (nonfinite && !(chk == T(0))) *nonfinite = 1;
}

// ---------------------------------------------------------------------------
// Reverse sweep: per step un-multiply the state by exp(-z), pull the adjoint
// back through the step, emit the increment gradient.
// (siglib/cpsig/cp_signature.h:1137-1187)
// ---------------------------------------------------------------------------
// LDS tile of the increment-gradient reduction: one row per (step-in-chunk, letter), one column per lane.
constexpr int kRedStride = 65;
// Reduction plan of one backward instance.  PAIR: before a step's per-letter sums go to the tile, the two
// half-waves exchange halves of the letter range (v_permlane32_swap) and add, so that lanes 0-31 hold letters
// 0 .. H-1 and lanes 32-63 letters H .. 2H-1 (H = ceil(d/2)), each already summed over the lane pair
// (lane, lane ^ 32).  The tile then has H rows per step instead of d: half the LDS writes and half the reads of
// the row sums.  Needs compile-time depth-1 letters (their pieces must already sit in the per-letter sums) and
// an LDS atomic that tolerates two lanes adding to one word (ds_add_f64).
template <typename T, int D, int TAIL, int K, bool ZL>
struct RedPlan {
    static constexpr int NG = D > 0 ? (D + K - 1) / K : 0;
    static constexpr bool PAIR = ZL && D > 0 && NG <= 3 && TAIL >= 2 && sizeof(T) == 8;
    static constexpr int kRows = int(16384 / (kRedStride * sizeof(T)));       // 31 (f64) / 63 (f32)
    // Wider paths get a tile of their own size holding a single step (up to 64 rows f64 / 128 rows f32, 33 KB per
    // wave): without it every lane of a wave would add into the same few LDS words.
    static constexpr int kRowsWide = 2 * kRows + 2;
    __host__ __device__ static constexpr int rows_per_step(int d) { return PAIR ? (d + 1) / 2 : d; }
    // steps per chunk of the tile; 0: the path is too wide for the tile
    __host__ __device__ static constexpr int steps(int d)
    {
        const int r = rows_per_step(d);
        return r > kRowsWide ? 0 : r > kRows ? 1 : (kRows / r > 8 ? 8 : kRows / r);
    }
    __host__ __device__ static constexpr int64_t tile_elems(int d) { return int64_t(steps(d)) * rows_per_step(d) * kRedStride; }
};

// lanes 0-31: lo[lane] + lo[lane + 32];  lanes 32-63: hi[lane - 32] + hi[lane]
__device__ __forceinline__ double pair_sum32(double lo, double hi)
{
    const auto r0 = __builtin_amdgcn_permlane32_swap(unsigned(__double2loint(lo)), unsigned(__double2loint(hi)), false, false);
    const auto r1 = __builtin_amdgcn_permlane32_swap(unsigned(__double2hiint(lo)), unsigned(__double2hiint(hi)), false, false);
    return __hiloint2double(int(r1[0]), int(r0[0])) + __hiloint2double(int(r1[1]), int(r0[1]));
}
__device__ __forceinline__ float pair_sum32(float lo, float) { return lo; }     // never used: PAIR needs 8-byte words

// Orders the LDS traffic of ONE wave: the hardware executes a wave's LDS operations in issue order, so lanes
// see each other's earlier writes and atomics without any wait; only the compiler has to be kept from moving
// memory operations across this point.  (A memory fence would also wait for the global atomics in flight.)
__device__ __forceinline__ void wave_lds_sync()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_wave_barrier();
    asm volatile("" ::: "memory");
}

// Add into an LDS word that only the calling lane touches between two wave_lds_sync() points (its own column
// of the reduction tile) or that several lanes may hit (the shared accumulator of the wide-path fallback).
// ds_add_f64 is fast; ds_add_f32 was measured several times slower than a plain read-add-write on gfx950, so
// the own-column case uses the latter for float.
template <typename T>
__device__ __forceinline__ void lds_add_shared(T* p, T v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ void lds_add(double* p, double v) { lds_add_shared(p, v); }
__device__ __forceinline__ void lds_add(float* p, float v) { *p += v; }
// sum over the 64 lanes of a wave, in every lane
template <typename T>
__device__ __forceinline__ T wave_sum(T v)
{
    for (int s = kWave >> 1; s; s >>= 1) v += __shfl_xor(v, s);
    return v;
}

template <typename T>
__device__ __forceinline__ void dev_add(T* p, T v)
{
    __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The forward sweep numbers its blocks per XCD (xcd_block): its HBM reads drop to the size of the path.  The backward
// keeps the dispatch order: with all waves of a path behind one L2 the atomic adds into a gradient row queue up in
// one cache channel instead of eight, which costs more (0.5 % of the sweep at batch 32, length 1000, d = 10, degree 5)
// than the saved re-reads of the increment rows give back.  -DSIGAMD_BWD_XCD=1 switches it on for measurements.
#ifndef SIGAMD_BWD_XCD
#define SIGAMD_BWD_XCD 0
#endif
constexpr bool kBwdXcd = SIGAMD_BWD_XCD != 0;

// LL: as in tree_fwd_kernel, and every item runs an even number of steps from an even first step (L and lseg even), so
// that the reverse sweep starts on an odd step; the gradients of the letters a step cannot move are left at zero
// (the raw path gradient never reads them).
template <typename T, int D, int N, int TAIL, int K, bool ZL, int LL = 0>
__global__ __launch_bounds__(kBlock) void tree_bwd_kernel(
    const T* __restrict__ inc, const T* __restrict__ sig, const T* __restrict__ gsig,
    T* __restrict__ dzinc, int64_t batch, int64_t L, int d_rt, int64_t sig_stride, int scalar,
    int use_lds, int nseg, int64_t lseg, int from_points)
{
    // `from_points` (staged kernels of narrow paths only): `inc` is the plain path [paths][L + 1][d] itself and the
    // increments are formed while they are staged.
    // `batch` counts (path, time segment) items: item vb = path * nseg + segment walks the increments of steps
    // [segment * lseg, min(L, (segment + 1) * lseg)) backwards, starting from the state `sig[vb]` (signature of the
    // path up to the segment's end) and the adjoint `gsig[vb]` (gradient w.r.t. that state).  nseg == 1 is the
    // plain whole-path sweep.  Steps are counted locally (count - 1 .. 0) so that every wave-level decision stays
    // uniform; when several items share a wave all of them run lseg steps and the surplus steps of a shorter
    // (last) segment, which walk into the previous segment, are dead: their gradient is not emitted.
    using Tr = Tree<T, D, N, TAIL, K>;
    using Ad = TreeAdj<T, D, N, TAIL, K>;
    using Cx = LaneCtx<T, D, N, TAIL, K>;
    constexpr int M = Tr::M;
    extern __shared__ double lds_raw[];
    T* lds = reinterpret_cast<T*>(lds_raw);

    Cx cx;
    cx.init(d_rt, batch, kBwdXcd);
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
    // Every lane adds its pieces of a step into its own column of an LDS tile
    // [row = step-in-chunk * d + letter][lane] (row stride 65: writers and summing lanes both hit distinct
    // banks; own column: no atomic ever collides).  When the chunk is full each (row, column segment) is
    // summed by one lane and added to dz[path][step][letter] in HBM.  Column segments: the lanes of one path
    // when several whole paths share the wave, else two halves of the wave.  Paths too wide for the tile
    // (d > 64 in f64, d > 128 in f32; up to half of that the tile holds several steps, beyond it a single one) fall
    // back to a per-wave accumulator updated with LDS atomics.
    const int lane = threadIdx.x & (kWave - 1);
    const int wave_in_block = threadIdx.x >> 6;
    constexpr bool WIDE = Cx::WIDE;
    using Plan = RedPlan<T, D, TAIL, K, ZL>;
    constexpr bool PAIR = Plan::PAIR;
    const int CH = Plan::steps(d);
    const int RS = Plan::rows_per_step(d);      // tile rows per step
    const bool tiled = CH > 0;
    const int slots = WIDE ? 1 : cx.G.ppw;
    T* wbuf = lds + int64_t(wave_in_block) * (tiled ? Plan::tile_elems(d) : use_lds == 2 ? int64_t(Plan::kRows) * kRedStride : int64_t(slots) * d);
    T* acc = wbuf + int64_t(cx.id.slot) * d;
    const int nsg = slots > 1 ? slots : 2;                    // column segments per row
    const int seg_cnt = slots > 1 ? int(cx.G.lpp) : kWave / 2; // lanes per segment
    if (!tiled && use_lds == 1) {
        for (int e = lane; e < slots * d; e += kWave) wbuf[e] = T(0);
        wave_lds_sync();
    }
    int64_t b_first;
    {
        const int64_t wave = xcd_block(kBwdXcd) * kWavesPerBlock + wave_in_block;
        b_first = (slots > 1) ? wave * slots : (wave / cx.G.wpp);
    }
    // path and first step of an item (whole paths skip the divisions)
    auto split_item = [&](int64_t vb, int64_t& pth, int64_t& s0) {
        if (nseg == 1) {
            pth = vb;
            s0 = 0;
        } else {
            pth = vb / nseg;
            s0 = (vb - pth * nseg) * lseg;
        }
    };
    // this lane's item
    int64_t it_path, it_t0;
    split_item(cx.id.b, it_path, it_t0);
    const int64_t it_ns = nseg == 1 ? L : (L - it_t0 < lseg) ? L - it_t0 : lseg;
    const int64_t count = nseg == 1 ? L : slots > 1 ? lseg : it_ns;       // steps this wave runs (wave-uniform)
    // element index of dz[path][step of local index 0][0] of an item, and its number of live steps
    auto item_base = [&](int64_t vb, int64_t& live) -> int64_t {
        int64_t pth, s0;
        split_item(vb, pth, s0);
        live = (L - s0 < lseg) ? L - s0 : lseg;
        return (pth * L + s0 + live - count) * d;
    };
    const int64_t lane_base = (it_path * L + it_t0 + it_ns - count) * d;
    // when the wave serves one item every lane holds that item, so its base is the lane's
    const int64_t wave_base = lane_base;
    int cs = 0;                     // steps already written into the current chunk
    int64_t t_chunk = count - 1;    // local step held by chunk slot 0
    // The tile is flushed when `limit` steps sit in it.  The first chunk takes the remainder of count / CH, so that
    // all later chunks are full and the last flush falls on the last step: the test is one 32-bit compare per step.
    int limit = tiled ? (count % CH == 0 ? CH : int(count % CH)) : 0;
    // The four waves of a block run in step, and four flushes at once queue up in the one LDS unit of the CU.  Each
    // wave therefore closes its first chunk at a different fill (the last chunk is then partial and flushed after the
    // sweep), which spreads the flushes of a block over the steps: 2 % of the sweep at batch 32, length 1000, d = 10.
    if (tiled) limit = (limit - 1 + (wave_in_block * CH) / kWavesPerBlock) % CH + 1;

    auto reduce_chunk = [&](int n_slots) {
        wave_lds_sync();
        const int items = n_slots * RS * nsg;
        for (int it = lane; it < items; it += kWave) {
            const int sg = it % nsg, r = it / nsg;
            const T* src = wbuf + r * kRedStride + sg * seg_cnt;
            T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
            if (seg_cnt == kWave / 2) {
#pragma unroll
                for (int i = 0; i < kWave / 2; i += 4) {
                    s0 += src[i];
                    s1 += src[i + 1];
                    s2 += src[i + 2];
                    s3 += src[i + 3];
                }
            } else {
                int i = 0;
                for (; i + 4 <= seg_cnt; i += 4) {
                    s0 += src[i];
                    s1 += src[i + 1];
                    s2 += src[i + 2];
                    s3 += src[i + 3];
                }
                for (; i < seg_cnt; ++i) s0 += src[i];
            }
            T sum = (s0 + s1) + (s2 + s3);
            const int slot = r / RS, j = r % RS;
            const int64_t tl = t_chunk - slot;      // local step of this row
            if constexpr (PAIR) {
                const int letter = j + RS * sg;      // the two halves of a row belong to different letters
                if (letter < d && b_first < batch) dev_add(&dzinc[wave_base + tl * d + letter], sum);
            } else if (slots > 1) {
                const int64_t bb = b_first + sg;
                if (bb < batch) {
                    int64_t live;
                    const int64_t base = item_base(bb, live);
                    if (tl >= count - live) dev_add(&dzinc[base + tl * d + j], sum);
                }
            } else {
                sum += __shfl_xor(sum, 1);      // the two halves of a row sit in neighbouring lanes
                if (sg == 0 && b_first < batch) dev_add(&dzinc[wave_base + tl * d + j], sum);
            }
        }
        wave_lds_sync();
    };

    // PAIR: word of each chain letter within a step's rows (row and half-wave of the letter, column of this lane in that half)
    int chain_off[M];
    if constexpr (PAIR) {
        constexpr int H = (Tr::DD + 1) / 2;
#pragma unroll
        for (int l = 0; l < M; ++l) {
            const int hi = cx.p[l] >= H ? 1 : 0;
            chain_off[l] = (cx.p[l] - H * hi) * kRedStride + 32 * hi + (lane & 31);
        }
    }
    auto do_step = [&](const typename Tr::Inc& z, int64_t t, auto g0c, auto posc) {
        constexpr int G0 = decltype(g0c)::value;
        constexpr bool FOLD = Ad::template kFoldDepth1<G0>;     // depth-1 pieces already sit in dz.dj
        // position 0 of the reverse sweep is the last step of an even-length range: an odd step
        using Act = std::conditional_t<LL == 0, AllLetters, LeadLagLetters<Tr::DD, 1 - decltype(posc)::value, G0>>;
        typename Tr::Chain unmul;
        S.template fwd_step<Act, true>(z, &unmul);     // state before the step
        typename Ad::DInc dz;
#pragma unroll
        for (int j = 0; j < Tr::DD; ++j) dz.dj[j] = T(0);
#pragma unroll
        for (int a = 0; a < K; ++a) dz.da[a] = T(0);
#pragma unroll
        for (int l = 0; l < M; ++l) dz.dc[l] = T(0);
        A.template pullback<G0, Act>(S, z, dz, Tr::kLockstep ? &unmul : nullptr);

        if (tiled) {
            // Idle lanes need no predicate: their adjoints were loaded as zero, so every piece they produce is zero.
            T* col = wbuf + cs * (RS * kRedStride) + lane;
            if constexpr (PAIR) {
                static_assert(!PAIR || FOLD, "pairing needs the depth-1 pieces folded into the per-letter sums");
                constexpr int H = (Tr::DD + 1) / 2;
#pragma unroll
                for (int r = 0; r < H; ++r)
                    col[r * kRedStride] = pair_sum32(dz.dj[r], r + H < Tr::DD ? dz.dj[r + H < Tr::DD ? r + H : 0] : T(0));
                T* base = wbuf + cs * (RS * kRedStride);
#pragma unroll
                for (int l = 0; l < M; ++l) lds_add_shared(&base[chain_off[l]], dz.dc[l]);
            } else if constexpr (TAIL >= 2) {
#pragma unroll
                for (int j = 0; j < Tr::DD; ++j) col[j * kRedStride] = dz.dj[j];
            } else {
                for (int j = 0; j < d; ++j) col[j * kRedStride] = T(0);
            }
            // depth-1 letters and chain letters go into the lane's own column; LDS executes a wave's operations in order
            if constexpr (!PAIR) {
                if constexpr (!FOLD) {
#pragma unroll
                    for (int a = 0; a < K; ++a)
                        if (cx.a0 + a < d) lds_add(&col[(cx.a0 + a) * kRedStride], dz.da[a]);
                }
#pragma unroll
                for (int l = 0; l < M; ++l) lds_add(&col[cx.p[l] * kRedStride], dz.dc[l]);
            }
            ++cs;
            if (cs == limit) {
                reduce_chunk(cs);
                t_chunk -= cs;
                cs = 0;
                limit = CH;
            }
        } else if (use_lds == 2) {
            // Paths too wide for a tile that holds a whole step (wave serves one item): the letters of the step pass
            // through a tile of kRows rows in groups.  Per group every lane clears its own column, adds the pieces
            // whose letters fall into the group (own column: no two lanes ever meet), and the rows are summed and
            // added to the gradient as in reduce_chunk.
            constexpr int RW = Plan::kRows;
            T* col = wbuf + lane;
            const bool live_step = t >= count - it_ns;
            for (int base = 0; base < d; base += RW) {
                const int nrow = d - base < RW ? d - base : RW;
                for (int r = 0; r < nrow; ++r) col[r * kRedStride] = T(0);
                auto emit = [&](int letter, T v) {
                    if (letter >= base && letter < base + nrow) lds_add(&col[(letter - base) * kRedStride], v);
                };
                if constexpr (TAIL >= 2) {
#pragma unroll
                    for (int j = 0; j < Tr::DD; ++j) emit(j, dz.dj[j]);
                }
                if constexpr (!FOLD) {
#pragma unroll
                    for (int a = 0; a < K; ++a)
                        if (cx.a0 + a < d) emit(cx.a0 + a, dz.da[a]);
                }
#pragma unroll
                for (int l = 0; l < M; ++l) emit(cx.p[l], dz.dc[l]);
                wave_lds_sync();
                for (int it = lane; it < nrow * 2; it += kWave) {
                    const int sg = it & 1, r = it >> 1;
                    const T* src = wbuf + r * kRedStride + sg * (kWave / 2);
                    T s0 = T(0), s1 = T(0), s2 = T(0), s3 = T(0);
#pragma unroll
                    for (int i = 0; i < kWave / 2; i += 4) {
                        s0 += src[i];
                        s1 += src[i + 1];
                        s2 += src[i + 2];
                        s3 += src[i + 3];
                    }
                    T sum = (s0 + s1) + (s2 + s3);
                    sum += __shfl_xor(sum, 1);          // the two halves of a row sit in neighbouring lanes
                    if (sg == 0 && live_step && b_first < batch) dev_add(&dzinc[wave_base + t * d + base + r], sum);
                }
                wave_lds_sync();
            }
        } else {
            T* grow_t = dzinc + lane_base + t * d;
            const bool live_step = t >= count - it_ns;
            if (use_lds) {
                if (active) {
#pragma unroll
                    for (int a = 0; a < K; ++a)
                        if (cx.a0 + a < d) lds_add_shared(&acc[cx.a0 + a], dz.da[a]);
                    if constexpr (TAIL >= 2) {
#pragma unroll
                        for (int j = 0; j < Tr::DD; ++j) lds_add_shared(&acc[j], dz.dj[j]);
                    }
#pragma unroll
                    for (int l = 0; l < M; ++l) lds_add_shared(&acc[cx.p[l]], dz.dc[l]);
                }
                wave_lds_sync();
                for (int e = lane; e < slots * d; e += kWave) {
                    const T v = wbuf[e];
                    wbuf[e] = T(0);
                    const int64_t bb = b_first + e / d;
                    if (bb < batch) {
                        int64_t live;
                        const int64_t base = item_base(bb, live);
                        if (t >= count - live) dev_add(&dzinc[base + t * d + e % d], v);
                    }
                }
                wave_lds_sync();
            } else if (active && live_step) {
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

    // row of the item's last step; point-fed: the point that step starts from
    const T* row = from_points ? inc + (it_path * (L + 1) + it_t0 + it_ns - 1) * d : inc + (it_path * (L + 2) + it_t0 + it_ns) * d;
    if constexpr (ZL) {
        static_assert(WIDE, "staged increments need the wide layout");
        T* lds_wave = lds + kWavesPerBlock * Plan::tile_elems(Tr::DD) + wave_in_block * IncRing<T, Tr::DD, -1>::ELEMS;
        constexpr int NG = (Tr::DD + K - 1) / K;
        const bool points = IncRing<T, Tr::DD, -1>::kPoints && from_points != 0;
        if constexpr (NG <= 3) {
            static_for<0, NG - 1>([&](auto gc) {
                if (cx.id.g == decltype(gc)::value)
                    sweep_staged<-1, decltype(gc)::value * K, Tr>(cx, row, count - 1, count, lds_wave, do_step, points);
            });
        } else {
            sweep_staged<-1, -1, Tr>(cx, row, count - 1, count, lds_wave, do_step, points);
        }
    } else {
        sweep_direct<-1, false, Cx, typename Tr::Inc>(cx, row, count - 1, count, do_step);
    }
    if (tiled && cs > 0) reduce_chunk(cs);      // what the staggered first chunk left over
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
    int time_aug, int lead_lag, T time_step, int scalar, int* __restrict__ nonfinite)
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
        if (nonfinite && not_finite(v)) *nonfinite = 1;
    }
}

// effective dimension 1: level k = Delta^k / k!
template <typename T>
__global__ __launch_bounds__(kBlock) void dim_one_fwd_kernel(
    const T* __restrict__ path, T* __restrict__ out, int64_t batch, int64_t len_raw, int degree, int scalar,
    int* __restrict__ nonfinite)
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
        if (nonfinite && not_finite(v)) *nonfinite = 1;      // once a level is not finite, so is the last
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
// Index arithmetic of the coefficient-per-thread kernels.  Word indices are decoded with divisions by the path
// dimension only; with 32-bit indices (every index below 2^31, the usual case) that division is a multiply-high
// and a shift by host-computed constants, with 64-bit indices a plain division.
// ---------------------------------------------------------------------------
template <typename I>
struct DivBy;
template <>
struct DivBy<uint32_t> {
    uint32_t d, mul, shr;
    __host__ explicit DivBy(uint64_t den) : d(uint32_t(den)), mul(0), shr(0)
    {
        if (d > 1) {
            uint32_t lg = 0;
            while ((uint64_t(1) << lg) < d) ++lg;
            const uint32_t p = 31 + lg;
            mul = uint32_t(((uint64_t(1) << p) + d - 1) / d);
            shr = p - 32;
        }
    }
    __device__ __forceinline__ uint32_t quot(uint32_t n) const { return d == 1 ? n : __umulhi(n, mul) >> shr; }   // n < 2^31
};
template <>
struct DivBy<uint64_t> {
    uint64_t d;
    __host__ explicit DivBy(uint64_t den) : d(den) {}
    __device__ __forceinline__ uint64_t quot(uint64_t n) const { return n / d; }
};

// test hook: nonzero makes launch_indexed pick 64-bit indices whatever the size (defined in sig_api.hip)
extern std::atomic<int> g_force_wide_index;

// calls f(index type tag, 2-D grid): grid.x covers `per_item` work items of one batch entry, grid.y the batch
template <typename F>
void launch_indexed(uint64_t max_index, uint64_t per_item, uint64_t batch, F&& f)
{
    uint64_t gx = (per_item + kBlock - 1) / kBlock;
    if (gx < 1) gx = 1;
    if (gx > (1u << 20)) gx = 1u << 20;
    const uint64_t gy = batch < 65535 ? (batch < 1 ? 1 : batch) : 65535;
    const dim3 grid{unsigned(gx), unsigned(gy), 1};
    if (max_index < (uint64_t(1) << 31) && !g_force_wide_index) f(uint32_t{}, grid);
    else f(uint64_t{}, grid);
}

// ---------------------------------------------------------------------------
// Increment pre-pass: z[b][t][c] of the (virtually) augmented path.
// lead-lag: even step moves the lead half, odd step the lag half; time is the
// last channel with constant spacing end_time / (len_eff - 1)
// (siglib/cpsig/cp_path.h:46-62,262-279; siglib/cusig/cu_signature.cu:146-166).
// Grid: x over the (L + 2) * d elements of one path, y over the paths; the only division is by d.
// ---------------------------------------------------------------------------
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void increments_kernel(
    const T* __restrict__ path, T* __restrict__ inc, int64_t batch, int64_t len_raw, int d_raw,
    int time_aug, int lead_lag, T time_step, T* __restrict__ zero_out, DivBy<I> dv)
{
    // zero_out (optional): the increment gradient [batch][L][d], cleared in the same launch; the backward
    // accumulates into it with atomics.
    // Layout [batch][L + 2][d]: row t + 1 holds the increment of step t; rows 0 and L + 1 are zero so
    // that the sweeps may prefetch one row past either end of a path without a bounds test.
    const I d = I(dv.d);
    const I L = I((lead_lag ? 2 * len_raw - 1 : len_raw) - 1);
    const I rows = L + 2;
    const I per = rows * d;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* x = path + b * len_raw * d_raw;
        T* o = inc + b * int64_t(per);
        T* zo = zero_out ? zero_out + b * int64_t(L) * int64_t(d) : nullptr;
        for (I e = I(blockIdx.x) * kBlock + threadIdx.x; e < per; e += I(gridDim.x) * kBlock) {
            const I row = dv.quot(e);
            const I c = e - row * d;
            T v;
            if (row == 0 || row == rows - 1) {
                v = T(0);
            } else {
                const I t = row - 1;
                if (time_aug && c == d - 1) {
                    // two separately rounded products, as the reference's GPU code forms it (siglib/cusig/cu_signature.cu:149-152)
                    v = mul_rn(T(t + 1), time_step) - mul_rn(T(t), time_step);
                } else if (!lead_lag) {
                    v = x[int64_t(t + 1) * d_raw + c] - x[int64_t(t) * d_raw + c];
                } else {
                    const I k = t >> 1;
                    const bool odd = t & 1;
                    if (c < I(d_raw)) v = odd ? x[int64_t(k + 1) * d_raw + c] - x[int64_t(k) * d_raw + c] : T(0);
                    else v = odd ? T(0) : x[int64_t(k + 1) * d_raw + (c - d_raw)] - x[int64_t(k) * d_raw + (c - d_raw)];
                }
            }
            o[e] = v;
            if (zo && e < L * d) zo[e] = T(0);
        }
    }
}

// ---------------------------------------------------------------------------
// Increment gradient -> raw path gradient.  Point i of the raw path receives
// +dz of every step that ends in it and -dz of every step that starts from it;
// with lead-lag, step 2k moves the lead half and step 2k+1 the lag half of
// raw segment k -> k+1; the time channel has no raw counterpart
// (siglib/cpsig/cp_signature.h:1189-1201, siglib/cusig/cu_path_transforms.cu:129-147).
// ---------------------------------------------------------------------------
// `clear` (optional): clear_count elements of another buffer are set to zero by the same launch: the increment-gradient
// accumulator the NEXT backward call will add into (the two accumulators of a device take turns, so a call whose
// sweep forms its own increments needs no launch that clears one).
template <typename T>
__device__ __forceinline__ void clear_range(T* __restrict__ clear, int64_t count)
{
    if (!clear) return;
    const int64_t threads = int64_t(gridDim.x) * gridDim.y * kBlock;
    for (int64_t e = (int64_t(blockIdx.y) * gridDim.x + blockIdx.x) * kBlock + threadIdx.x; e < count; e += threads) clear[e] = T(0);
}

// Grid: x over the len_raw * d_raw elements of one path's gradient, y over the paths; the only division is by d_raw.
template <typename T, typename I>
__global__ __launch_bounds__(kBlock) void path_grad_kernel(
    const T* __restrict__ dzinc, T* __restrict__ out, int64_t batch, int64_t len_raw, int time_aug, int lead_lag,
    DivBy<I> dv, T* __restrict__ clear, int64_t clear_count)
{
    clear_range(clear, clear_count);
    const I d_raw = I(dv.d);
    const I d = (lead_lag ? 2 * d_raw : d_raw) + (time_aug ? 1 : 0);
    const int64_t L = (lead_lag ? 2 * len_raw - 1 : len_raw) - 1;
    const I per = I(len_raw) * d_raw;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* g = dzinc + b * L * int64_t(d);
        T* o = out + b * int64_t(per);
        for (I e = I(blockIdx.x) * kBlock + threadIdx.x; e < per; e += I(gridDim.x) * kBlock) {
            const int64_t i = int64_t(dv.quot(e));
            const int64_t c = int64_t(e) - i * int64_t(d_raw);
            T v = T(0);
            if (!lead_lag) {
                if (i > 0) v += g[(i - 1) * d + c];
                if (i < len_raw - 1) v -= g[i * d + c];
            } else {
                if (i > 0) v += g[(2 * (i - 1)) * d + d_raw + c] + g[(2 * (i - 1) + 1) * d + c];
                if (i < len_raw - 1) v -= g[(2 * i) * d + d_raw + c] + g[(2 * i + 1) * d + c];
            }
            o[e] = v;
        }
    }
}

// The same for plain paths (no augmentation) whose channel count is a multiple of V, with V elements per lane in one
// 16-byte access: there the increment gradient has the layout of the path and the kernel is a pure stream.
// Grid: x over the len_raw * d_raw / V vector elements of one path, y over the paths; dv divides by d_raw / V.
template <typename T, int V>
struct alignas(V * sizeof(T)) VecOf {
    T v[V];
};
template <typename T, typename I, int V>
__global__ __launch_bounds__(kBlock) void path_grad_vec_kernel(
    const T* __restrict__ dzinc, T* __restrict__ out, int64_t batch, int64_t len_raw, DivBy<I> dv,
    T* __restrict__ clear, int64_t clear_count)
{
    clear_range(clear, clear_count);
    using Vec = VecOf<T, V>;
    const I dvec = I(dv.d);
    const I per = I(len_raw) * dvec;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const Vec* g = reinterpret_cast<const Vec*>(dzinc) + b * (len_raw - 1) * int64_t(dvec);
        Vec* o = reinterpret_cast<Vec*>(out) + b * int64_t(per);
        for (I e = I(blockIdx.x) * kBlock + threadIdx.x; e < per; e += I(gridDim.x) * kBlock) {
            const int64_t i = int64_t(dv.quot(e));
            Vec r;
#pragma unroll
            for (int k = 0; k < V; ++k) r.v[k] = T(0);
            if (i > 0) {
                const Vec a = g[int64_t(e) - dvec];
#pragma unroll
                for (int k = 0; k < V; ++k) r.v[k] += a.v[k];
            }
            if (i < len_raw - 1) {
                const Vec a = g[e];
#pragma unroll
                for (int k = 0; k < V; ++k) r.v[k] -= a.v[k];
            }
            o[e] = r;
        }
    }
}

// level t (1-based) of coefficient r of a scalar-free signature row, its index w inside the level, the start
// `lo` and the size of the level
template <typename I>
struct WordPos {
    int t;
    I w, lo, size;
};
template <typename I>
__device__ __forceinline__ WordPos<I> word_pos(I r, I d)
{
    WordPos<I> p{1, 0, 0, d};
    while (r >= p.lo + p.size) { p.lo += p.size; p.size *= d; ++p.t; }
    p.w = r - p.lo;
    return p;
}

// ---------------------------------------------------------------------------
// Chen product C = A (x) B of two signatures per path (scalar terms implicit 1):
//   C_t[w] = A_t[w] + B_t[w] + sum_{k=1..t-1} A_k[w_1..w_k] * B_{t-k}[w_{k+1}..w_t]
// (siglib/cpsig/cp_sig_combine.h:35-66).  One thread per output coefficient; rows
// of A, B, C may have different strides and C may carry a leading scalar slot.
// ---------------------------------------------------------------------------

// LDS copies of the short levels of the two factors of a Chen product (chen_fan<.., LOW = true>): the block copies
// the first low_n coefficients of each row; barriers on both sides
template <typename T, typename I>
__device__ __forceinline__ void stage_low_levels(T* al, T* bl, const T* __restrict__ a, const T* __restrict__ bb, I low_n)
{
    __syncthreads();        // the row before is done with the copies
    for (I j = threadIdx.x; j < low_n; j += kBlock) {
        al[j] = a[j];
        bl[j] = bb[j];
    }
    __syncthreads();
}
// host: how many whole levels are copied, never the top level: at most 1536 coefficients per row (a longer copy costs a
// block more than its reads save).  Only for 8-byte elements (measured: +8..30 % for float64 rows, -9..+10 % for
// float32) and only when the launch keeps at least 4096 blocks after every thread has taken several items to amortise
// the copy (`blocks` = blocks of the launch at one item per thread).
extern std::atomic<int> g_chen_low_levels;      // test hook (defined in sig_api.hip): 0 = no copies, 1 = automatic, 2 = always
inline uint64_t chen_low_items_per_thread(uint64_t low_n, uint64_t blocks)
{
    const uint64_t per = (2 * low_n + 255) / 256;       // loads of the copy per thread
    const uint64_t room = g_chen_low_levels == 2 ? per : blocks / 4096;
    const uint64_t take = per < room ? per : room;
    return take < 1 ? 1 : (take > 8 ? 8 : take);
}
inline uint64_t chen_low_count(uint64_t d, uint64_t top, size_t elem_bytes, uint64_t blocks)
{
    if (!g_chen_low_levels || (g_chen_low_levels != 2 && (elem_bytes < 8 || blocks < 8192))) return 0;
    uint64_t n = 0, size = 1;
    for (uint64_t t = 1; t < top; ++t) {
        size *= d;
        if (n + size > 1536) break;
        n += size;
    }
    return n;
}

// The same sums for FAN outputs per thread: the words (a, rest) for FAN consecutive first letters a and one
// `rest` of t - 1 letters.  Every split pairs a prefix (a, head of rest) with a suffix that does not depend on a, so
// the suffix factor and all index arithmetic are shared by the outputs; consecutive threads hold consecutive `rest`
// and all loads and stores coalesce as in the one-output form, at about half the cache accesses per output (which is
// what bounds these kernels).  Work items of a row of `top` levels, level-major, then letter group, then rest:
// chen_items(d, top, FAN) = ceil(d / FAN) * (1 + d + .. + d^(top-1)).  f(r, sum) receives, for every output r, the sum
// over the proper splits, sum_{k=1..t-1} A_k[prefix] * B_{t-k}[suffix].
// FAN is chosen per dimension (with_chen_fan): the shared part of a thread costs about three outputs' worth, surplus
// letters of the last group do real work; d = 10 -> 5 (sig_combine at batch 1024, degree 5: 0.86 ms one output per
// thread, 0.72 ms FAN 4, 0.65 ms FAN 5).
constexpr int kChenFanMax = 8;
inline int chen_fan_for(uint64_t d)
{
    int best = 1;
    uint64_t best_cost = ~uint64_t(0);
    for (int f = 1; f <= kChenFanMax; ++f) {
        if (uint64_t(f) > d) break;
        const uint64_t cost = (d + f - 1) / f * (3 + f);
        if (cost <= best_cost) { best = f; best_cost = cost; }
    }
    return best;
}
// calls f(IntC<FAN>{}) with the fan of dimension d
template <typename F>
void with_chen_fan(uint64_t d, F&& f)
{
    switch (chen_fan_for(d)) {
        case 1: f(IntC<1>{}); break;
        case 2: f(IntC<2>{}); break;
        case 3: f(IntC<3>{}); break;
        case 4: f(IntC<4>{}); break;
        case 5: f(IntC<5>{}); break;
        case 6: f(IntC<6>{}); break;
        case 7: f(IntC<7>{}); break;
        default: f(IntC<8>{}); break;
    }
}
inline uint64_t chen_items(uint64_t d, uint64_t top, int fan)
{
    uint64_t words = 0, size = 1;       // 1 + d + .. + d^(top-1): below the coefficient count of the row, which the caller checked
    for (uint64_t t = 0; t < top; ++t) {
        words += size;
        size *= d;
    }
    return (d + fan - 1) / fan * words;
}
// work item -> level t, the start `lo` of that level in a scalar-free row, size = d^(t-1), the first letter a0 of the
// item's group and the index `rest` of the remaining t - 1 letters
template <typename I>
struct FanItem {
    int t;
    I lo, size, a0, rest;
};
template <typename I, int FAN>
__device__ __forceinline__ FanItem<I> fan_item(I item, I d)
{
    const I groups = (d + FAN - 1) / FAN;
    FanItem<I> it{1, 0, 1, 0, 0};
    I first = 0;                        // first item of level t
    while (item >= first + groups * it.size) {
        first += groups * it.size;
        it.lo += it.size * d;
        it.size *= d;
        ++it.t;
    }
    const I local = item - first;
    const I g = local / it.size;
    it.rest = local - g * it.size;
    it.a0 = g * FAN;
    return it;
}

// LOW: the first `low_n` coefficients of both rows (whole levels) also sit in LDS at `al` / `bl` (stage_low_levels) and
// are read from there: most factors of a product belong to the short levels, and with all of them coming from memory
// these kernels are bound by the rate of vector memory instructions, not by bandwidth (texture addresser ~90 % busy).
template <typename T, typename I, int FAN, bool LOW = false, typename F>
__device__ __forceinline__ void chen_fan(const T* __restrict__ a, const T* __restrict__ bb, I item, const DivBy<I>& dv, F&& f,
                                         const T* al = nullptr, const T* bl = nullptr, I low_n = 0)
{
    constexpr int kChenFan = FAN;
    const I d = I(dv.d);
    const FanItem<I> fi = fan_item<I, FAN>(item, d);
    const int t = fi.t;
    const I lo = fi.lo, size = fi.size, a0 = fi.a0, rest = fi.rest;
    T acc[kChenFan];
#pragma unroll
    for (int i = 0; i < kChenFan; ++i) acc[i] = T(0);
    I pre = rest, suf = 0, pw = 1;      // head of rest, suffix, d^(letters in the suffix)
    I lev = size * d, a_lo = lo;        // size and start of level k + 1 of A
    I b_lo = 0;                         // start of level t - k of B
    for (int k = t - 1; k >= 1; --k) {
        const I q = dv.quot(pre);
        suf += (pre - q * d) * pw;
        pw *= d;
        pre = q;
        lev = dv.quot(lev);             // d^k
        a_lo -= lev;
        const I st = dv.quot(lev);      // d^(k-1): distance between the prefixes of consecutive first letters
        T bv;
        if (LOW && b_lo + suf < low_n) bv = bl[b_lo + suf];
        else bv = bb[b_lo + suf];
        if (LOW && a_lo < low_n) {      // a whole level: the same for every lane of the block but at level borders
            const T* ap = al + a_lo + pre;
#pragma unroll
            for (int i = 0; i < kChenFan; ++i) {
                const I letter = a0 + i < d ? a0 + i : d - 1;
                acc[i] = fmadd(ap[letter * st], bv, acc[i]);
            }
        } else {
            const T* ap = a + a_lo + pre;
#pragma unroll
            for (int i = 0; i < kChenFan; ++i) {
                const I letter = a0 + i < d ? a0 + i : d - 1;      // surplus outputs shadow the last letter
                acc[i] = fmadd(ap[letter * st], bv, acc[i]);
            }
        }
        b_lo += pw;
    }
#pragma unroll
    for (int i = 0; i < kChenFan; ++i)
        if (a0 + i < d) f(lo + (a0 + i) * size + rest, acc[i]);
}

template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void sig_combine_kernel(
    const T* __restrict__ A, const T* __restrict__ B, T* __restrict__ C, int64_t batch, DivBy<I> dv,
    I items /* chen_items(d, degree, FAN) */, int64_t a_stride, int64_t b_stride, int64_t c_stride,
    int a_off, int b_off, int c_off, I low_n /* chen_low_count: dynamic LDS of 2 * low_n entries; 0 = none */)
{
    extern __shared__ double chen_low_raw[];
    T* al = reinterpret_cast<T*>(chen_low_raw);
    T* bl = al + low_n;
    for (int64_t b = blockIdx.y; b < batch; b += gridDim.y) {
        const T* a = A + b * a_stride + a_off;
        const T* bb = B + b * b_stride + b_off;
        T* c = C + b * c_stride;
        if (low_n) stage_low_levels(al, bl, a, bb, low_n);
        for (I it = I(blockIdx.x) * kBlock + threadIdx.x; it < items; it += I(gridDim.x) * kBlock) {
            if (low_n) chen_fan<T, I, FAN, true>(a, bb, it, dv, [&](I r, T sum) { c[c_off + r] = a[r] + bb[r] + sum; }, al, bl, low_n);
            else chen_fan<T, I, FAN>(a, bb, it, dv, [&](I r, T sum) { c[c_off + r] = a[r] + bb[r] + sum; });
            if (c_off && it == 0) c[0] = T(1);
        }
    }
}

// One doubling step of two scans over the segment signatures seg[path][g] (rows of sig_len coefficients, nseg per
// path): the running products from the left, X[g] = seg[0] (x) .. (x) seg[g], and the products of everything to the
// right, Z[g] = seg[g+1] (x) .. (x) seg[nseg-1] (the unit for the last segment; a unit is a zero row).  A step with
// shift s maps X[g] <- X[g-s] (x) X[g] and Z[g] <- Z[g] (x) Z[g+s], rows beyond either end being units; after the
// steps s = 1, 2, 4, .. < nseg both scans are complete.  In the first step (z_first) the rows of Z are read from the
// segment signatures one row further right.  Work item: (scan, path, g) on blockIdx.y, coefficients on blockIdx.x.
template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void chen_scan_step_kernel(
    const T* __restrict__ xsrc, const T* __restrict__ zsrc, T* __restrict__ xdst, T* __restrict__ zdst, int64_t paths,
    int nseg, int shift, int z_first, DivBy<I> dv, I sig_len, I items /* chen_items(d, degree, FAN) */)
{
    const int64_t rows = paths * nseg;
    for (int64_t y = blockIdx.y; y < 2 * rows; y += gridDim.y) {
        const bool right = y >= rows;
        const int64_t row = right ? y - rows : y;
        const int g = int(row % nseg);
        const T* a = nullptr;
        const T* bb = nullptr;
        T* c = (right ? zdst : xdst) + row * int64_t(sig_len);
        if (!right) {
            if (g - shift >= 0) a = xsrc + (row - shift) * int64_t(sig_len);
            bb = xsrc + row * int64_t(sig_len);
        } else {
            const int g0 = g + z_first;      // row holding Z[g]
            if (g0 < nseg) a = zsrc + (row + z_first) * int64_t(sig_len);
            if (g0 + shift < nseg) bb = zsrc + (row + z_first + shift) * int64_t(sig_len);
        }
        if (a && bb) {
            for (I it = I(blockIdx.x) * kBlock + threadIdx.x; it < items; it += I(gridDim.x) * kBlock)
                chen_fan<T, I, FAN>(a, bb, it, dv, [&](I r, T sum) { c[r] = a[r] + bb[r] + sum; });
        } else {
            for (I r = I(blockIdx.x) * kBlock + threadIdx.x; r < sig_len; r += I(gridDim.x) * kBlock)
                c[r] = a ? a[r] : bb ? bb[r] : T(0);
        }
    }
}

// One halving step of the ordered product of m rows per path: dst[path][j] = row[2j] (x) row[2j+1] for j < m / 2.
// The rows of a path are `src_rows` consecutive rows of `src`, followed, when `carry` is set, by one more row that
// lives elsewhere (carry + path * carry_path_stride).  An unpaired last row is not copied: the caller hands it to the
// next step as that step's carry.  dst rows have their own stride between paths and may carry a leading scalar slot,
// so the last step (m = 2) can write the caller's signature directly.
template <typename T, typename I, int FAN>
__global__ __launch_bounds__(kBlock) void chen_fold_step_kernel(
    const T* __restrict__ src, int src_rows, const T* __restrict__ carry, int64_t carry_path_stride, T* __restrict__ dst,
    int64_t paths, int m, int64_t dst_path_stride, int dst_off, DivBy<I> dv, I sig_len,
    I items /* chen_items(d, degree, FAN) */, int* __restrict__ nonfinite)
{
    const int pairs = m / 2;
    for (int64_t y = blockIdx.y; y < paths * pairs; y += gridDim.y) {
        const int64_t path = y / pairs;
        const int j = int(y % pairs);
        const T* a = src + (path * src_rows + 2 * j) * int64_t(sig_len);
        const T* bb = (2 * j + 1 == src_rows) ? carry + path * carry_path_stride : a + int64_t(sig_len);
        T* c = dst + path * dst_path_stride + int64_t(j) * int64_t(sig_len);
        for (I it = I(blockIdx.x) * kBlock + threadIdx.x; it < items; it += I(gridDim.x) * kBlock) {
            chen_fan<T, I, FAN>(a, bb, it, dv, [&](I r, T sum) {
                const T v = a[r] + bb[r] + sum;
                c[dst_off + r] = v;
                if (nonfinite && not_finite(v)) *nonfinite = 1;
            });
            if (dst_off && it == 0) c[0] = T(1);
        }
    }
}

}  // namespace sigamd
