// Register-resident prefix-tree kernels for the truncated path signature on gfx950.
//
// One lane owns a word prefix p of length M = N - TAIL together with
//   * the chain  S_1[p_1], S_2[p_1 p_2], ..., S_M[p]           (M values, recomputed
//     redundantly by every lane that shares part of the prefix), and
//   * a slice of the subtree below p: at subtree depth 1 the K letters
//     a0 .. a0+K-1 (a0 = K * group), below that all D letters, down to depth TAIL.
// All of it lives in VGPRs for the whole sweep over the path; HBM sees the
// increments (read through the scalar cache when a wave serves one path) and
// one final store.  The update of a coefficient only reads coefficients of its
// own prefixes, so lanes never exchange signature state.
//
// The arithmetic is the reference's Horner step
// (siglib/cpsig/cp_signature.h:464-499 forward, :1137-1187 backward) regrouped
// per word; see the comments on fwd_step / pullback below.
//
// D > 0: compile-time path dimension.  D == 0: run-time dimension (TAIL must be 1), lanes of several groups and
// paths packed into waves.  D == -1: run-time dimension in the wide layout (every wave serves one letter group of
// one path; needs d^M >= 48, which the host checks before it picks such a kernel).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace sigamd {

constexpr int kWave = 64;
constexpr int kBlock = 256;
constexpr int kWavesPerBlock = kBlock / kWave;

__host__ __device__ constexpr int64_t ipow64(int64_t b, int e)
{
    int64_t r = 1;
    for (int i = 0; i < e; ++i) r *= b;
    return r;
}

// 1 / k.  Reciprocals that are no inline constant of the instruction set (k > 2) are handed out in scalar registers,
// set once per kernel: as a literal, a multiply-add by such a number has to overwrite its addend, and the compiler
// then copies the addend first whenever it lives on (one more issue slot per use).
template <typename T>
__device__ __forceinline__ T rcp(int k)
{
    T v = T(1) / T(k);
#ifndef SIGAMD_LITERAL_RCP
    if (k > 2 && (k & (k - 1)) == 0) asm("" : "+s"(v));
#endif
    return v;
}

// the increment as a step sees it: NEG steps run on the negated increment.  Negating an operand where it is used costs
// nothing (an operand modifier), while products of the increment itself stay common to a step and its negated twin.
template <bool NEG, typename T>
__device__ __forceinline__ T sgn(T x) { return NEG ? -x : x; }

template <typename T>
__device__ __forceinline__ T fmadd(T a, T b, T c) { return __builtin_fma(a, b, c); }
template <>
__device__ __forceinline__ float fmadd<float>(float a, float b, float c) { return __builtin_fmaf(a, b, c); }

// Launch geometry shared by host and device.
//   wide:   the prefixes of one path fill whole waves; lane order is group-major
//           with the prefix range padded to a multiple of 64, so path index and
//           group are wave-uniform (increments become scalar loads).
//   packed: lanes of one path are contiguous (prefix-major, group fastest);
//           if a path needs <= 64 lanes several whole paths share a wave,
//           otherwise a path takes ceil(lanes/64) waves.
struct TreeGeom {
    int64_t P;          // number of prefixes D^M
    int ng;             // groups at subtree depth 1
    int wide;
    int64_t p_pad;      // wide: P rounded up to 64
    int64_t lpp;        // lanes per path (wide: ng * p_pad; packed: ng * P)
    int ppw;            // packed, lpp <= 64: whole paths per wave, else 1
    int64_t wpp;        // waves per path when a path spans waves, else 1
};

__host__ __device__ inline TreeGeom make_geom(int d, int m, int k, bool allow_wide)
{
    TreeGeom g;
    g.P = ipow64(d, m);
    g.ng = (d + k - 1) / k;
    g.wide = allow_wide && g.P >= 48;   // must agree with the kernel's compile-time choice
    if (g.wide) {
        g.p_pad = (g.P + kWave - 1) / kWave * kWave;
        g.lpp = g.ng * g.p_pad;
        g.ppw = 1;
        g.wpp = g.lpp / kWave;
    } else {
        g.p_pad = g.P;
        g.lpp = g.ng * g.P;
        if (g.lpp <= kWave) { g.ppw = int(kWave / g.lpp); g.wpp = 1; }
        else { g.ppw = 1; g.wpp = (g.lpp + kWave - 1) / kWave; }
    }
    return g;
}

inline int64_t total_waves(const TreeGeom& g, int64_t batch)
{
    if (g.ppw > 1) return (batch + g.ppw - 1) / g.ppw;
    return batch * g.wpp;
}

struct LaneId {
    int64_t b;      // path index
    int64_t q;      // prefix number in [0, P)
    int g;          // group
    int slot;       // index of the path inside its wave (packed, several paths per wave)
    bool active;
};

// The dispatcher deals the blocks of a grid to the 8 XCDs in turn (block p runs on XCD p % 8), and every XCD has an
// L2 of its own.  Renumbering the blocks so that each XCD works on one contiguous range keeps the waves of a path
// (which read the same increment rows and add into the same gradient rows) behind one L2: the rows are fetched from
// HBM once instead of once per XCD, and the atomics of a row meet in one cache.
constexpr uint32_t kXcds = 8;
__device__ __forceinline__ int64_t xcd_block(bool on = true)
{
    const uint32_t nb = gridDim.x, p = blockIdx.x;
    if (!on) return p;
    const uint32_t x = p % kXcds, base = nb / kXcds, rem = nb % kXcds;
    return int64_t(x) * base + (x < rem ? x : rem) + p / kXcds;
}

// The same for 2-D grids (x: work inside a row, y: rows), which are dispatched x-fastest: each XCD takes whole rows
// one after the other, so a row that several blocks read again and again is fetched into one L2 only.
struct Block2 {
    uint32_t x, y;
};
__device__ __forceinline__ Block2 xcd_block_2d()
{
    const uint32_t gx = gridDim.x;
    const uint64_t nb = uint64_t(gx) * gridDim.y, p = uint64_t(blockIdx.y) * gx + blockIdx.x;
    const uint64_t x = p % kXcds, base = nb / kXcds, rem = nb % kXcds;
    const uint64_t l = x * base + (x < rem ? x : rem) + p / kXcds;
    return Block2{uint32_t(l % gx), uint32_t(l / gx)};
}

template <bool WIDE>
__device__ __forceinline__ LaneId lane_id(const TreeGeom& G, int64_t batch, bool xcd)
{
    LaneId id;
    const int lane = threadIdx.x & (kWave - 1);
    int64_t wave = xcd_block(xcd) * kWavesPerBlock + (threadIdx.x >> 6);
    id.slot = 0;
    if constexpr (WIDE) {
        // wave-uniform quantities are forced into SGPRs
        const uint32_t wlo = __builtin_amdgcn_readfirstlane(uint32_t(wave));
        const uint32_t whi = __builtin_amdgcn_readfirstlane(uint32_t(uint64_t(wave) >> 32));
        wave = int64_t((uint64_t(whi) << 32) | wlo);
        id.b = wave / G.wpp;
        const int64_t w = wave % G.wpp;
        const int64_t wpg = G.p_pad / kWave;
        id.g = int(w / wpg);
        id.q = (w % wpg) * kWave + lane;
        id.active = id.b < batch && id.q < G.P;
    } else {
        int64_t lip;
        if (G.ppw > 1) {
            id.slot = lane / int(G.lpp);
            id.b = wave * G.ppw + id.slot;
            lip = lane % int(G.lpp);
            id.active = id.slot < G.ppw && id.b < batch;
        } else {
            id.b = wave / G.wpp;
            lip = (wave % G.wpp) * kWave + lane;
            id.active = id.b < batch && lip < G.lpp;
        }
        id.q = lip / G.ng;
        id.g = int(lip % G.ng);
    }
    return id;
}

// ---------------------------------------------------------------------------
// Per-lane signature state and the Horner step on it.
// ---------------------------------------------------------------------------
// Which letters of a step's increment can be non-zero, known at compile time.
// Lead-lag paths move one half of the channels per step (siglib/cpsig/cp_path.h:262-279): with d_raw = D / 2 raw
// channels, steps of odd index move the letters [0, d_raw), steps of even index the letters [d_raw, 2 d_raw), and a
// time channel (the last letter when D is odd) moves in every step.  A forward step that knows this skips the
// multiply-adds by the zero letters - they would add exactly nothing - which is close to half of its work.
// G0: first depth-1 letter of the lane's group when known at compile time, else -1 (depth 1 is then treated as dense).
struct AllLetters {
    static constexpr int G0 = -1;
    __host__ __device__ static constexpr bool on(int) { return true; }
};
template <int D, int PARITY, int G0_>
struct LeadLagLetters {
    static constexpr int G0 = G0_;
    __host__ __device__ static constexpr bool on(int letter)
    {
        const int d_raw = D / 2;
        if ((D & 1) && letter == D - 1) return true;                        // time
        return PARITY ? letter < d_raw : (letter >= d_raw && letter < 2 * d_raw);
    }
};

template <typename T, int D, int N, int TAIL, int K>
struct Tree {
    static_assert(TAIL >= 1 && TAIL < N, "need a non-empty prefix and a non-empty subtree");
    static_assert(D > 0 || TAIL == 1, "run-time dimension supports depth-1 subtrees only");
    static constexpr int M = N - TAIL;
    static constexpr int DD = D > 0 ? D : 1;
    static constexpr int TAIL_ = TAIL;
    static constexpr int K_ = K;
    // subtree depth e (1-based) holds K * D^(e-1) values starting at off(e)
    __host__ __device__ static constexpr int cnt(int e) { return K * int(ipow64(DD, e - 1)); }
    __host__ __device__ static constexpr int off(int e)
    {
        int o = 0;
        for (int i = 1; i < e; ++i) o += cnt(i);
        return o;
    }
    static constexpr int SUB = off(TAIL + 1);

    T c[M];       // chain: c[l-1] = S_l[p_1..p_l]
    T s[SUB];     // subtree slice

    // Letters seen by one step: z[j] for the compile-time letters below subtree
    // depth 1, zs[a] = z[a0 + a] for the depth-1 slice, pz[l] = z[p_{l+1}].
    struct Inc {
        T z[DD];
        T zs[K];
        T pz[M];
    };

    // Horner values along the prefix: for target level t (2 <= t <= N) and chain depth l + 1 (l < depth(t))
    //   u[t][0] = z[p_1]/t + S_1[p_1];   u[t][l] = u[t][l-1] * z[p_{l+1}] / (t-l) + S_{l+1}[p_1..p_{l+1}]
    // (siglib/cpsig/cp_signature.h:464-499 regrouped per word).
    __host__ __device__ static constexpr int depth(int t) { return t - 1 < M ? t - 1 : M; }
    // Short prefixes: the chains of all target levels are evaluated first, in lockstep over the depth, so that
    // consecutive instructions belong to different levels.  Long prefixes have enough levels in flight for the
    // scheduler to overlap one level's chain with another level's subtree by itself; they go level by level,
    // which keeps fewer values alive.
    static constexpr bool kLockstep = M <= 4;
    struct Chain {
        T u[N + 1][M];
        T q[N + 1][M];      // q[t][l] = z[p_{l+1}] / (t - l), l >= 1: the scaled prefix letters the chains multiply by
    };

    // Keeps the instruction scheduler from re-serialising what the source interleaves: the compiler's machine
    // model lets dependent FP64 FMAs issue back to back, while the hardware stalls them when a SIMD holds a
    // single wave (measured: a few percent of a sweep).
    __device__ __forceinline__ static void pin() { __builtin_amdgcn_sched_barrier(0); }

    // All chains of one step in lockstep over the depth; every value is computed from the state before the step.
    // reuse (may be null): the chains of the step with the negated increment taken from the state AFTER that step, i.e.
    // from this state's successor.  Its value at depth t - 1 of target level t is the integral of the level's node
    // along the segment, the same number from either end, so those entries are taken over instead of computed
    // (levels up to kReuseMax, the ones the negated step evaluates).
    static constexpr int kReuseMax = M + 1 < N - 1 ? M + 1 : N - 1;
    template <bool NEG = false>
    __device__ __forceinline__ void chain_all(const Inc& in, Chain& ch, const Chain* reuse = nullptr) const
    {
#pragma unroll
        for (int l = 0; l < M; ++l) {
#pragma unroll
            for (int t = l + 2; t <= N; ++t) {
                if (reuse && t == l + 2 && t <= kReuseMax) ch.u[t][l] = reuse->u[t][l];
                // the sign goes to the chain value: the negated product would be folded into a constant of the other sign
                else ch.u[t][l] = (l == 0) ? fmadd(sgn<NEG>(in.pz[0]), rcp<T>(t), c[0]) : fmadd(sgn<NEG>(ch.u[t][l - 1]), ch.q[t][l], c[l]);
            }
            if (l + 1 < M) {
#pragma unroll
                for (int t = l + 3; t <= N; ++t) {
                    if (reuse && t <= N - 1) {
                        ch.q[t][l + 1] = reuse->q[t][l + 1];        // the negated step's products: the same numbers
                    } else {
                        ch.q[t][l + 1] = in.pz[l + 1] * rcp<T>(t - l - 1);
                    }
                }
            }
            pin();
        }
    }

    // Level-by-level form, used for long prefixes: U_t at chain depth `depth` (1 <= depth <= min(t-1, M)):
    //   U(1) = z[p_1]/t + S_1[p_1];  U(l+1) = U(l) * z[p_{l+1}] / (t-l) + S_{l+1}[..]
    // All intermediate values are returned in u[0..depth).
    template <int t, int depth, bool NEG = false>
    __device__ __forceinline__ void chain_u(const Inc& in, T (&u)[M > 0 ? M : 1]) const
    {
        u[0] = fmadd(sgn<NEG>(in.pz[0]), rcp<T>(t), c[0]);
#pragma unroll
        for (int l = 1; l < depth; ++l) u[l] = fmadd(u[l - 1] * rcp<T>(t - l), sgn<NEG>(in.pz[l]), c[l]);
    }

    template <int E>
    __device__ __forceinline__ static T zc(const Inc& in, int ch)
    {
        if constexpr (E == 1) return in.zs[ch];
        else return in.z[ch];
    }

    // Descend the subtree for target depth I (target level t = M + I).  `upar`
    // is U_t of the parent (depth E-1 node `pidx`; the root is the prefix p).
    // ACT: the letters that can be non-zero in this step; the others' multiply-adds are left out
    template <int E, typename ACT>
    __host__ __device__ static constexpr bool letter_on(int ch)
    {
        if (E == 1) return ACT::G0 < 0 || ACT::on(ACT::G0 + ch);
        return ACT::on(ch);
    }
    template <int E, int I, typename ACT = AllLetters, bool NEG = false>
    __device__ __forceinline__ void fwd_desc(const Inc& in, T upar, int pidx)
    {
        constexpr int NCH = (E == 1) ? K : DD;
        if constexpr (E == I) {
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch)
                if (letter_on<E, ACT>(ch))
                    s[off(E) + pidx * NCH + ch] = fmadd(upar, sgn<NEG>(zc<E>(in, ch)), s[off(E) + pidx * NCH + ch]);
        } else {
            // the children's Horner values first, their consumers afterwards: no FMA directly follows its producer
            const T ur = upar * rcp<T>(I - E + 1);
            T uc[NCH];
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch)
                uc[ch] = letter_on<E, ACT>(ch) ? fmadd(ur, sgn<NEG>(zc<E>(in, ch)), s[off(E) + pidx * NCH + ch]) : s[off(E) + pidx * NCH + ch];
            if constexpr (NCH >= 4) pin();      // narrow fans: the regions between pins would be too small to fill
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch) fwd_desc<E + 1, I, ACT, NEG>(in, uc[ch], pidx * NCH + ch);
        }
    }

    // subtree target levels t, t-1, ..., M+1: descending, so that every read of a shallower depth still sees the
    // value from before the step
    template <int t, typename ACT = AllLetters, bool NEG = false>
    __device__ __forceinline__ void fwd_subtree(const Inc& in, const Chain& ch)
    {
        if constexpr (t > M) {
            fwd_desc<1, t - M, ACT, NEG>(in, ch.u[t][M - 1], 0);
            fwd_subtree<t - 1, ACT, NEG>(in, ch);
        }
    }

    template <int t, typename ACT = AllLetters, bool NEG = false>
    __device__ __forceinline__ void fwd_level(const Inc& in)
    {
        if constexpr (t == 1) {
            c[0] += sgn<NEG>(in.pz[0]);
        } else if constexpr (t <= M) {
            T u[M > 0 ? M : 1];
            chain_u<t, t - 1, NEG>(in, u);
            c[t - 1] = fmadd(u[t - 2], sgn<NEG>(in.pz[t - 1]), c[t - 1]);
        } else {
            T u[M > 0 ? M : 1];
            chain_u<t, M, NEG>(in, u);
            fwd_desc<1, t - M, ACT, NEG>(in, u[M - 1], 0);
        }
        if constexpr (t > 1) fwd_level<t - 1, ACT, NEG>(in);
    }

    // S <- S (x) exp(z): target levels in descending order so that every read of
    // a lower level still sees the value from before the step
    // (siglib/cpsig/cp_signature.h:464-499).
    // NEG: the step with the negated increment, S <- S (x) exp(-z) (the reverse sweep's un-multiply).
    // keep (lockstep chains only, may be null): receives the chains of this step, for TreeAdj::pullback to take over.
    template <typename ACT = AllLetters, bool NEG = false>
    __device__ __forceinline__ void fwd_step(const Inc& in, Chain* keep = nullptr)
    {
        if constexpr (!kLockstep) {
            fwd_level<N, ACT, NEG>(in);
            return;
        }
        Chain ch;
        chain_all<NEG>(in, ch);
        fwd_subtree<N, ACT, NEG>(in, ch);
#pragma unroll
        for (int t = M; t >= 2; --t) c[t - 1] = fmadd(ch.u[t][t - 2], sgn<NEG>(in.pz[t - 1]), c[t - 1]);
        c[0] += sgn<NEG>(in.pz[0]);
        if (keep) *keep = ch;
    }
};

// Adjoint state of one lane: partial adjoints of the shared chain (seeded in one
// lane only; the recursion is linear in the adjoint so the partials add up) and
// the adjoints of the owned subtree slice.
template <typename T, int D, int N, int TAIL, int K>
struct TreeAdj {
    using Tr = Tree<T, D, N, TAIL, K>;
    static constexpr int M = Tr::M;
    static constexpr int DD = Tr::DD;
    T gc[M];
    T gs[Tr::SUB];

    // Per-step increment gradient pieces of this lane:
    //   dj[j]  -> letter j            (compile-time letters, subtree depth >= 2)
    //   da[a]  -> letter a0 + a       (subtree depth 1)
    //   dc[l]  -> letter p_{l+1}      (chain)
    // top: the prefix word's Horner value towards the top level (depth-1 subtrees only): da[a] = gs[a] * top, for
    // sweeps that form these products elsewhere
    struct DInc {
        T dj[DD];
        T da[K];
        T dc[M];
        T top;
    };
    // depth-1 pieces can join dj in registers when the depth-1 letters are compile-time constants and dj is in use
    template <int G0>
    static constexpr bool kFoldDepth1 = G0 >= 0 && TAIL >= 2;

    // Post-order pullback through the subtree for target depth I.  Returns the
    // adjoint flowing into the parent's Horner value ("reduced" in
    // siglib/cpsig/cp_signature.h:1158-1180); children adjoints are the upstream
    // gradient at depth I and the recursion's return values above it.
    // G0 >= 0: the lane's depth-1 letters are the compile-time letters G0 .. G0+K-1 and their pieces are added
    // to dj[G0 + a] straight away (da stays untouched); G0 < 0: the letters are only known at run time -> da.
    // ACT: the letters that can be non-zero in this step.  A letter that cannot move contributes nothing to the
    // contractions with z, and its increment gradient is never read (the raw path gradient takes, per step, only the
    // channels that step moves), so both of its multiply-adds are left out; the adjoint itself still flows through it.
    template <int E, int I, int G0, typename ACT = AllLetters>
    __device__ __forceinline__ T bwd_desc(const Tr& S, const typename Tr::Inc& in, DInc& dz, T upar, int pidx)
    {
        constexpr int NCH = (E == 1) ? K : DD;
        const T sc = rcp<T>(I - E + 1);
        const T v = (I - E + 1 == 1) ? upar : upar * sc;
        if constexpr (TAIL == 1) dz.top = v;
        T red = T(0);
        T uc[NCH];
        if constexpr (E < I) {
            // the children's Horner values first, their consumers afterwards
#pragma unroll
            for (int ch = 0; ch < NCH; ++ch)
                uc[ch] = Tr::template letter_on<E, ACT>(ch) ? fmadd(v, Tr::template zc<E>(in, ch), S.s[Tr::off(E) + pidx * NCH + ch])
                                                            : S.s[Tr::off(E) + pidx * NCH + ch];
            if constexpr (NCH >= 4) Tr::pin();
        }
#pragma unroll
        for (int ch = 0; ch < NCH; ++ch) {
            const int ci = Tr::off(E) + pidx * NCH + ch;
            T adj;
            if constexpr (E == I) {
                adj = gs[ci];
            } else {
                adj = bwd_desc<E + 1, I, G0, ACT>(S, in, dz, uc[ch], pidx * NCH + ch);
                gs[ci] += adj;
            }
            if (!Tr::template letter_on<E, ACT>(ch)) continue;
            if constexpr (E == 1 && kFoldDepth1<G0>) {
                if (G0 + ch < DD) dz.dj[(G0 + ch < DD) ? G0 + ch : 0] = fmadd(adj, v, dz.dj[(G0 + ch < DD) ? G0 + ch : 0]);
            } else if constexpr (E == 1) {
                dz.da[ch] = fmadd(adj, v, dz.da[ch]);
            } else {
                dz.dj[ch] = fmadd(adj, v, dz.dj[ch]);
            }
            red = fmadd(adj, Tr::template zc<E>(in, ch), red);
        }
        return (I - E + 1 == 1) ? red : red * sc;
    }

    // Walk the adjoint `adj` of chain node `from` (1-based depth) up to the root.
    template <int t, int from>
    __device__ __forceinline__ void chain_up(const typename Tr::Inc& in, DInc& dz, const T (&u)[M > 0 ? M : 1], T adj)
    {
#pragma unroll
        for (int l = from - 1; l >= 1; --l) {
            // node p_1..p_l, child letter p_{l+1}
            const T sc = rcp<T>(t - l);
            const T v = u[l - 1] * sc;
            dz.dc[l] = fmadd(adj, v, dz.dc[l]);
            adj = adj * in.pz[l] * sc;
            gc[l - 1] += adj;
        }
        dz.dc[0] = fmadd(adj, rcp<T>(t), dz.dc[0]);
    }

    template <int t, int G0, typename ACT = AllLetters>
    __device__ __forceinline__ void bwd_level(const Tr& S, const typename Tr::Inc& in, DInc& dz)
    {
        if constexpr (t == 1) {
            dz.dc[0] += gc[0];
        } else if constexpr (t <= M) {
            T u[M > 0 ? M : 1];
            S.template chain_u<t, t - 1>(in, u);
            chain_up<t, t>(in, dz, u, gc[t - 1]);
        } else {
            T u[M > 0 ? M : 1];
            S.template chain_u<t, M>(in, u);
            const T red = bwd_desc<1, t - M, G0, ACT>(S, in, dz, u[M - 1], 0);
            gc[M - 1] += red;
            chain_up<t, M>(in, dz, u, red);
        }
        if constexpr (t < N) bwd_level<t + 1, G0, ACT>(S, in, dz);
    }

    // subtree target levels M+1 .. N in ascending order: the upstream adjoint of depth I is consumed before
    // deeper targets add into it.  a[t] receives the adjoint flowing into the prefix node's Horner value.
    template <int t, int G0, typename ACT = AllLetters>
    __device__ __forceinline__ void bwd_subtree(const Tr& S, const typename Tr::Inc& in, DInc& dz,
                                                const typename Tr::Chain& ch, T (&a)[N + 1])
    {
        if constexpr (t <= N) {
            a[t] = bwd_desc<1, t - M, G0, ACT>(S, in, dz, ch.u[t][M - 1], 0);
            bwd_subtree<t + 1, G0, ACT>(S, in, dz, ch, a);
        }
    }

    // Pull the adjoint back through one step S_after = S (x) exp(z), where S is
    // the state BEFORE the step.  Target levels ascend so that the adjoint of
    // level t is consumed before higher levels add into it
    // (siglib/cpsig/cp_signature.h:1147-1187).
    // unmul (lockstep chains only, may be null): the chains of the step with the negated increment that produced S
    // from its successor (Tree::fwd_step<ACT, true>), see Tree::chain_all.
    template <int G0 = -1, typename ACT = AllLetters>
    __device__ __forceinline__ void pullback(const Tr& S, const typename Tr::Inc& in, DInc& dz,
                                             const typename Tr::Chain* unmul = nullptr)
    {
        if constexpr (!Tr::kLockstep) {
            bwd_level<1, G0, ACT>(S, in, dz);
            return;
        }
        typename Tr::Chain ch;
        S.template chain_all<false>(in, ch, unmul);
        // Every target level t reads the adjoint of its own chain node as it was before the step and adds into
        // shallower nodes only, so all starting adjoints are taken first and the walks to the root run in
        // lockstep over the depth (consecutive instructions belong to different levels).
        T a[N + 1];
        const T g1 = gc[0];
#pragma unroll
        for (int t = 2; t <= M; ++t) a[t] = gc[t - 1];
        bwd_subtree<M + 1, G0, ACT>(S, in, dz, ch, a);
#pragma unroll
        for (int t = M + 1; t <= N; ++t) gc[M - 1] += a[t];
#pragma unroll
        for (int l = M - 1; l >= 1; --l) {
            // node p_1..p_l, child letter p_{l+1}; levels t > l pass through it
#pragma unroll
            for (int t = l + 1; t <= N; ++t) {
                const T v = ch.u[t][l - 1] * rcp<T>(t - l);
                dz.dc[l] = fmadd(a[t], v, dz.dc[l]);
                a[t] = a[t] * (in.pz[l] * rcp<T>(t - l));
            }
            if (l == 1) {
                // the root letter's piece starts from the level-1 adjoint as it was before the step: taken here, ahead
                // of the sums into that adjoint, it needs no copy
                dz.dc[0] += gc[0];
#pragma unroll
                for (int t = 2; t <= N; ++t) dz.dc[0] = fmadd(a[t], rcp<T>(t), dz.dc[0]);
            }
#pragma unroll
            for (int t = l + 1; t <= N; ++t) gc[l - 1] += a[t];
            Tr::pin();
        }
        if constexpr (M == 1) {
            dz.dc[0] += g1;
#pragma unroll
            for (int t = 2; t <= N; ++t) dz.dc[0] = fmadd(a[t], rcp<T>(t), dz.dc[0]);
        }
    }
};

}  // namespace sigamd
