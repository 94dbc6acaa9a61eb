// Streaming form of the adjoint of the Chen product C = A (x) B (siglib/cpsig/cp_sig_combine.h:126-176): the rows of
// dC are read once per factor, in memory order.
//
//   dA_k[u] = dC_k[u] + sum_{m >= 1} sum_{v in d^m} dC_{k+m}[u v] * B_m[v]     sums over the FAST index of dC
//   dB_t[w] = dC_t[w] + sum_{k >= 1} sum_{u in d^k} dC_{k+t}[u w] * A_k[u]     sums over the SLOW index of dC
//
// Left factor (chen_adjoint_left_kernel): a block owns c consecutive words p of length np = N - mt and, with them, the
// coefficients p* of every level np .. N: one contiguous piece per level, c d^j entries, copied to LDS with coalesced
// loads.  Every dA_k[p s] with k >= np sums over pieces that are all in LDS (rows of length d^m, with B_1 .. B_mt
// beside them in LDS), so it is complete when the block stores it: no atomics.  Words shorter than np collect one
// partial sum per block and level through an atomic; their terms from levels <= np come from the item-per-word kernel
// run on the signature truncated at level np, launched first.
//
// Right factor (chen_adjoint_right_kernel): a lane owns a word f of length qe (64 consecutive f per wave, so that
// every load of dC is one contiguous 64-entry piece) and walks the words w of length 1 .. N - qe in front of it
// depth first, last letter outermost.  dC[w f] adds into the accumulator of every suffix w[i:] f on the path of the
// walk, weighted with A[w[:i]]: a wave-uniform operand.  dB_t with t >= qe is complete when the walk leaves its
// node; shorter words (t < qe) collect per-lane partial sums with lane-dependent weights A[w f[:qe-t]] and receive
// them through atomics at the end; their terms from levels < qe again come from the item-per-word kernel.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>

#include "sig_kernels.h"

namespace sigamd {

constexpr int kStreamMaxLevels = 32;
constexpr int kRightMaxRel = 4;      // depth of the walk in front of a lane's word
constexpr int kRightMaxLow = 7;      // levels below the length of a lane's word
constexpr int kLeftMaxTile = 12;     // levels of a block's LDS pieces

struct StreamLevels {
    uint32_t lo[kStreamMaxLevels + 2];      // start of level t in a scalar-free row, t = 1 .. degree + 1
    uint32_t pw[kStreamMaxLevels + 2];      // d^i while it fits 31 bits
};

static inline bool fill_stream_levels(StreamLevels& lv, uint64_t d, uint64_t degree);

struct RightPlan {
    int degree, qe, rel;        // rel = degree - qe
    uint32_t d, words;          // words = d^qe
    StreamLevels lv;
};

struct LeftPlan {
    int degree, mt, np, upb;    // levels in LDS below the owned words, length of the owned words, units per block
    uint32_t d, c, units, xs, bs;
    uint32_t xoff[kLeftMaxTile + 2];        // piece of level np + j inside the LDS copy of dC (multiples of 64)
    uint32_t boff[kLeftMaxTile + 2];        // level m of B inside its LDS copy: (d^m - d) / (d - 1)
    uint32_t gsz[kLeftMaxTile + 1];         // lanes that share a row sum at relative level j: a power of two <= 64, or the block
    StreamLevels lv;
};

// loads / stores with a wave-uniform base and a per-lane byte offset (one scalar pair + one 32-bit lane register)
template <typename T>
__device__ __forceinline__ T load_at(const T* base, uint32_t byte_off)
{
    return *reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + byte_off);
}
template <typename T>
__device__ __forceinline__ void store_at(T* base, uint32_t byte_off, T v)
{
    *reinterpret_cast<T*>(reinterpret_cast<char*>(base) + byte_off) = v;
}

template <typename T, int QL>
struct RightLane {
    const T* g;
    const T* a;
    T* out;
    uint32_t f, fo;                     // the lane's word and its byte offset
    bool live;
    int identity;
    uint32_t cq[QL > 0 ? QL : 1];       // f / d^t, t = 1 .. QL
    uint32_t cqo[QL > 0 ? QL : 1];      // the same as byte offsets
    T low[QL > 0 ? QL : 1];
    T acc[kRightMaxRel + 1];
    // folding with exp(z) as the right factor (FOLD): see chen_adjoint_right_kernel
    const T* z;                         // displacement of the row
    T* slot;                            // the lane's own d partial sums in LDS, kBlock entries apart
    T kacc[kRightMaxRel + 2];           // kacc[D]: sum over the visited children x of the node at depth D - 1
    T zp[kRightMaxRel + 1];             // product of z over the letters of the word at depth D
};

// 1 / level and 1 / level! of the words at depth D of the walk (level = qe + D)
template <typename T>
struct FoldScale {
    T inv_level[kRightMaxRel + 1];
    T inv_fact[kRightMaxRel + 1];
};

#ifndef SIGAMD_LEAF_BATCH
#define SIGAMD_LEAF_BATCH 5
#endif
constexpr int kLeafBatch = SIGAMD_LEAF_BATCH;       // loads of the deepest level that are in flight together

// visits the words (x w), x = 0 .. d-1, in front of the lane's word; `widx` is the index of w (length DEPTH - 1) and
// pfx[i] the index of its first i letters.  The deepest level issues its loads kLeafBatch at a time, and an inner
// level loads the entry of its next word before it walks below the current one: a lane's loads would otherwise
// pay their latency one after the other.
template <typename T, int QL, int REL, bool FOLD, int DEPTH>
__device__ __forceinline__ void right_descend(RightLane<T, QL>& L, const RightPlan& P, const FoldScale<T>& F, uint32_t widx,
                                              const uint32_t (&pfx)[kRightMaxRel + 1])
{
    const int lvl = P.qe + DEPTH;
    const T* grow = L.g + P.lv.lo[lvl];
    T* orow = L.out + P.lv.lo[lvl];
    if constexpr (DEPTH == REL) {
        [[maybe_unused]] T zq = T(0);
        if constexpr (FOLD) zq = L.zp[DEPTH - 1] * F.inv_fact[DEPTH];
        for (uint32_t x0 = 0; x0 < P.d; x0 += kLeafBatch) {
            T e[kLeafBatch];
            T w[QL > 0 ? QL : 1][kLeafBatch];
#pragma unroll
            for (int i = 0; i < kLeafBatch; ++i) {
                const uint32_t x = x0 + i;
                const uint32_t idx = x * P.lv.pw[DEPTH - 1] + widx;
                e[i] = T(0);
#pragma unroll
                for (int t = 1; t <= QL; ++t) w[t - 1][i] = T(0);
                if (x < P.d) {      // wave-uniform
                    if (L.live) e[i] = load_at(grow + idx * P.words, L.fo);
#pragma unroll
                    for (int t = 1; t <= QL; ++t) w[t - 1][i] = load_at(L.a + P.lv.lo[lvl - t] + idx * P.lv.pw[P.qe - t], L.cqo[t - 1]);
                }
            }
#pragma unroll
            for (int i = 0; i < kLeafBatch; ++i) {
                const uint32_t x = x0 + i;
                if (x < P.d) {
                    const uint32_t idx = x * P.lv.pw[DEPTH - 1] + widx;
#pragma unroll
                    for (int j = 0; j < DEPTH; ++j) {
                        const int len = DEPTH - j;      // first len letters of (x w)
                        const uint32_t head = x * P.lv.pw[len - 1] + pfx[len - 1];
                        L.acc[j] = fmadd(L.a[P.lv.lo[len] + head], e[i], L.acc[j]);
                    }
#pragma unroll
                    for (int t = 1; t <= QL; ++t) L.low[t - 1] = fmadd(w[t - 1][i], e[i], L.low[t - 1]);
                    if constexpr (FOLD) {
                        L.kacc[DEPTH] = fmadd(L.z[x] * F.inv_level[DEPTH], e[i], L.kacc[DEPTH]);
                        lds_add(L.slot + x * kBlock, e[i] * zq);
                    } else {
                        if (L.live && L.identity) store_at(orow + idx * P.words, L.fo, e[i]);
                    }
                }
            }
        }
    } else {
        T e = L.live ? load_at(grow + widx * P.words, L.fo) : T(0);      // x = 0
        for (uint32_t x = 0; x < P.d; ++x) {
            const uint32_t idx = x * P.lv.pw[DEPTH - 1] + widx;
            const uint32_t nxt = (x + 1 < P.d ? x + 1 : x) * P.lv.pw[DEPTH - 1] + widx;
            const T en = L.live ? load_at(grow + nxt * P.words, L.fo) : T(0);
            uint32_t np[kRightMaxRel + 1];
            np[0] = 0;
#pragma unroll
            for (int i = 1; i <= DEPTH; ++i) np[i] = x * P.lv.pw[i - 1] + pfx[i - 1];
            L.acc[DEPTH] = L.identity ? e : T(0);
            [[maybe_unused]] T zx = T(0);
            if constexpr (FOLD) {
                zx = L.z[x];
                L.zp[DEPTH] = L.zp[DEPTH - 1] * zx;
                L.kacc[DEPTH + 1] = T(0);
            }
#pragma unroll
            for (int j = 0; j < DEPTH; ++j) L.acc[j] = fmadd(L.a[P.lv.lo[DEPTH - j] + np[DEPTH - j]], e, L.acc[j]);
#pragma unroll
            for (int t = 1; t <= QL; ++t)
                L.low[t - 1] = fmadd(load_at(L.a + P.lv.lo[lvl - t] + idx * P.lv.pw[P.qe - t], L.cqo[t - 1]), e, L.low[t - 1]);
            right_descend<T, QL, REL, FOLD, DEPTH + 1>(L, P, F, idx, np);
            if constexpr (FOLD) {
                const T k = L.acc[DEPTH] + L.kacc[DEPTH + 1];
                L.kacc[DEPTH] = fmadd(zx * F.inv_level[DEPTH], k, L.kacc[DEPTH]);
                lds_add(L.slot + x * kBlock, k * (L.zp[DEPTH - 1] * F.inv_fact[DEPTH]));
            } else {
                if (L.live) store_at(orow + idx * P.words, L.fo, L.acc[DEPTH]);
            }
            e = en;
        }
    }
}

// grid: x over the waves of a row (4 per block), y over the rows
//
// FOLD: B = exp(z) and the caller wants dz, not dB (sig_join_backprop, siglib/cpsig/cp_sig_join.h:36-238).  With
//   K_t[v] = dB_t[v] + 1/(t+1) sum_a z[a] K_{t+1}[a v]      (K_N = dB_N)
// the adjoint of z -> exp(z) is dz[a] = sum_t 1/t! <K_t[a .], z^(t-1)>: a word's K sums over the letters in front of
// it, which is the order of the walk, so K_t for t > qe never leaves the lane.  Its terms go into dz here (a private
// LDS slot per lane and letter, summed over the wave at the end of a row, then one atomic per wave and letter);
// level qe of dB receives K_qe, levels below it dB itself as without FOLD, and the caller finishes with the adjoint of
// exp truncated at level qe on that row.  Needs identity = 1 and d * kBlock entries of dynamic LDS.
template <typename T, int QL, int REL, bool FOLD>
__global__ __launch_bounds__(kBlock) void chen_adjoint_right_kernel(
    const T* __restrict__ dC, T* __restrict__ dB, const T* __restrict__ A, int64_t batch, RightPlan P, int64_t stride,
    int off, int identity, int64_t dc_share, int64_t dc_stride, int dc_off, const T* __restrict__ Z, T* __restrict__ dz,
    FoldScale<T> F)
{
    extern __shared__ double right_lds_raw[];
    const Block2 blk = xcd_block_2d();
    const uint32_t wave = blk.x * kWavesPerBlock + (threadIdx.x >> 6);
    if (wave * kWave >= P.words) return;
    [[maybe_unused]] T* slot = reinterpret_cast<T*>(right_lds_raw) + threadIdx.x;
    if constexpr (FOLD)
        for (uint32_t x = 0; x < P.d; ++x) slot[x * kBlock] = T(0);
    for (int64_t b = blk.y; b < batch; b += gridDim.y) {
        RightLane<T, QL> L;
        L.g = dC + (b / dc_share) * dc_stride + dc_off;
        L.a = A + b * stride + off;
        L.out = dB + b * stride + off;
        const uint32_t f = wave * kWave + (threadIdx.x & (kWave - 1));
        L.live = f < P.words;
        L.f = L.live ? f : 0;
        L.fo = L.f * uint32_t(sizeof(T));
        L.identity = identity;
        if (off && f == 0) dB[b * stride] = T(0);
#pragma unroll
        for (int t = 1; t <= QL; ++t) {
            L.cq[t - 1] = L.f / P.lv.pw[t];
            L.cqo[t - 1] = L.cq[t - 1] * uint32_t(sizeof(T));
            L.low[t - 1] = T(0);
        }
        const uint32_t pos = P.lv.lo[P.qe] + L.f;
        const T e = L.live ? L.g[pos] : T(0);
        L.acc[0] = identity ? e : T(0);
#pragma unroll
        for (int t = 1; t <= QL; ++t) L.low[t - 1] = fmadd(L.a[P.lv.lo[P.qe - t] + L.cq[t - 1]], e, L.low[t - 1]);
        if constexpr (FOLD) {
            L.z = Z + b * int64_t(P.d);
            L.slot = slot;
            T prod = T(1);
            uint32_t rest = L.f;
            for (int i = 0; i < P.qe; ++i) {
                const uint32_t q = rest / P.d;
                prod *= L.z[rest - q * P.d];
                rest = q;
            }
            L.zp[0] = prod;
            L.kacc[1] = T(0);
        }
        const uint32_t root[kRightMaxRel + 1] = {0, 0, 0, 0, 0};
        right_descend<T, QL, REL, FOLD, 1>(L, P, F, 0u, root);
        if constexpr (FOLD) {
            L.acc[0] += L.kacc[1];
            for (uint32_t x = 0; x < P.d; ++x) {
                const T v = wave_sum(slot[x * kBlock]);
                slot[x * kBlock] = T(0);
                if ((threadIdx.x & (kWave - 1)) == 0) dev_add(dz + b * int64_t(P.d) + x, v);
            }
        }
        if (L.live) {
            L.out[pos] = L.acc[0];
#pragma unroll
            for (int t = 1; t <= QL; ++t) dev_add(L.out + P.lv.lo[t] + (L.f - L.cq[t - 1] * P.lv.pw[t]), L.low[t - 1]);
        }
    }
}

// sum over one row of the left factor's gradient: entries r d^m + v of the pieces j + m, m = 1 .. mt - j, times B_m[v];
// `lane` of `G` lanes takes every G-th entry
template <typename T>
__device__ __forceinline__ T left_row_sum(const LeftPlan& P, const T* X, const T* Bl, int j, uint32_t r, uint32_t lane, uint32_t G)
{
    T a0 = T(0), a1 = T(0), a2 = T(0), a3 = T(0);
    for (int m = 1; m <= P.mt - j; ++m) {
        const uint32_t len = P.lv.pw[m];
        const T* xr = X + P.xoff[j + m] + r * len;
        const T* br = Bl + P.boff[m];
        uint32_t v = lane;
        for (; v + 3 * G < len; v += 4 * G) {       // four independent LDS reads in flight
            const T x0 = xr[v], x1 = xr[v + G], x2 = xr[v + 2 * G], x3 = xr[v + 3 * G];
            const T b0 = br[v], b1 = br[v + G], b2 = br[v + 2 * G], b3 = br[v + 3 * G];
            a0 = fmadd(x0, b0, a0);
            a1 = fmadd(x1, b1, a1);
            a2 = fmadd(x2, b2, a2);
            a3 = fmadd(x3, b3, a3);
        }
        for (; v < len; v += G) a0 = fmadd(xr[v], br[v], a0);
    }
    return (a0 + a1) + (a2 + a3);
}

// grid: x over groups of `upb` units of a row, y over the rows; dynamic LDS: (xs + bs) entries.  KX * kBlock >= xs:
// a thread holds entries tid + kBlock i of a unit's LDS image in registers, loaded (all loads in flight together)
// while the block still works on the unit before.
template <typename T, int KX>
__global__ __launch_bounds__(kBlock) void chen_adjoint_left_kernel(
    const T* __restrict__ dC, T* __restrict__ dA, const T* __restrict__ B, int64_t batch, LeftPlan P, int64_t stride,
    int off, int identity, int64_t dc_share, int64_t dc_stride, int dc_off)
{
    extern __shared__ __align__(16) unsigned char chen_lds[];
    T* X = reinterpret_cast<T*>(chen_lds);
    T* Bl = X + P.xs;
    __shared__ T part[3][kWavesPerBlock];      // [0]: long level np - 1, [2]: block-wide row sums
    const uint32_t tid = threadIdx.x;
    const int N = P.degree, mt = P.mt, np = P.np;
    const int nreg = np - 1 < 1 ? np - 1 : 1;        // the long level np - 1 is summed from registers
    const Block2 blk = xcd_block_2d();
    const uint32_t u0 = blk.x * uint32_t(P.upb);
    const uint32_t u1 = u0 + uint32_t(P.upb) < P.units ? u0 + uint32_t(P.upb) : P.units;
    if (u0 >= u1) return;
    for (int64_t b = blk.y; b < batch; b += gridDim.y) {
        const T* g = dC + (b / dc_share) * dc_stride + dc_off;
        const T* other = B + b * stride + off;
        T* out = dA + b * stride + off;
        if (off && blk.x == 0 && tid == 0) dA[b * stride] = T(0);
        // Entry z = tid + kBlock i of a unit's LDS image.  Pieces start at multiples of 64 entries, so the 64 entries
        // a wave handles in slot i lie in one piece: the piece and every address base are wave-uniform, and a lane adds
        // the same byte offset to all of them.
        T rx[KX], rb1[KX];
        const uint32_t lane_off = (tid & (kWave - 1)) * uint32_t(sizeof(T));
        const uint32_t wave0 = __builtin_amdgcn_readfirstlane(tid & ~uint32_t(kWave - 1));
        auto slot_piece = [&](int i, uint32_t& rel0) {      // piece of slot i and the piece-relative index of lane 0
            const uint32_t zw = wave0 + uint32_t(kBlock) * i;
            int j = mt;
            while (zw < P.xoff[j]) --j;
            rel0 = zw - P.xoff[j];
            return j;
        };
        auto fetch = [&](uint32_t unit) {
            const uint32_t p0 = unit * P.c;
            const uint32_t rem1 = nreg >= 1 ? p0 % P.lv.pw[1] : 0;
#pragma unroll
            for (int i = 0; i < KX; ++i) {
                rx[i] = T(0);
                rb1[i] = T(0);
                if (wave0 + uint32_t(kBlock) * i < P.xs) {
                    uint32_t rel0;
                    const int j = slot_piece(i, rel0);
                    if (rel0 + (tid & (kWave - 1)) < P.c * P.lv.pw[j]) {
                        rx[i] = load_at(g + P.lv.lo[np + j] + p0 * P.lv.pw[j] + rel0, lane_off);
                        if (j >= 1 && nreg >= 1) rb1[i] = load_at(other + P.lv.lo[1 + j] + rem1 * P.lv.pw[j] + rel0, lane_off);
                    }
                }
            }
        };
        fetch(u0);
        __syncthreads();                                                        // the row before is done with Bl
        for (uint32_t z = tid; z < P.bs; z += kBlock) Bl[z] = other[z];        // levels 1 .. mt open the row
        for (uint32_t unit = u0; unit < u1; ++unit) {
            const uint32_t p0 = unit * P.c;
            __syncthreads();                                                    // readers of the unit before are done
            T s1 = T(0);
            {
                T* top = out + P.lv.lo[N] + p0 * P.lv.pw[mt];                  // the top level has no sum
#pragma unroll
                for (int i = 0; i < KX; ++i) {
                    const uint32_t zw = wave0 + uint32_t(kBlock) * i;
                    if (zw < P.xs) {
                        X[zw + (tid & (kWave - 1))] = rx[i];                    // padding receives zeros
                        if (zw >= P.xoff[mt] && zw - P.xoff[mt] + (tid & (kWave - 1)) < P.c * P.lv.pw[mt])
                            if (identity) store_at(top + (zw - P.xoff[mt]), lane_off, rx[i]);
                        s1 = fmadd(rx[i], rb1[i], s1);
                    }
                }
            }
            if (nreg >= 1) {
                for (int s = kWave >> 1; s; s >>= 1) s1 += __shfl_xor(s1, s);
                if ((tid & (kWave - 1)) == 0) part[0][tid >> 6] = s1;
            }
            __syncthreads();
            if (nreg >= 1 && tid == 0) {
                T sum = part[0][0];
                for (int w = 1; w < kWavesPerBlock; ++w) sum += part[0][w];
                dev_add(out + P.lv.lo[np - 1] + p0 / P.lv.pw[1], sum);
            }
            if (unit + 1 < u1) fetch(unit + 1);
            // words p s, |s| = j < mt: all their terms are in LDS
            for (int j = 0; j < mt; ++j) {
                const uint32_t G = P.gsz[j], rows = P.c * P.lv.pw[j];
                T* dst = out + P.lv.lo[np + j] + p0 * P.lv.pw[j];
                if (G <= uint32_t(kWave)) {
                    const uint32_t lane_g = tid & (G - 1), step = kBlock / G;
                    for (uint32_t r = tid / G; r < rows; r += step) {
                        T acc = left_row_sum(P, X, Bl, j, r, lane_g, G);
                        for (uint32_t s = G >> 1; s; s >>= 1) acc += __shfl_xor(acc, int(s));
                        if (lane_g == 0) dst[r] = (identity ? X[P.xoff[j] + r] : T(0)) + acc;
                    }
                } else {      // few long rows: the whole block sums one row
                    for (uint32_t r = 0; r < rows; ++r) {
                        T acc = left_row_sum(P, X, Bl, j, r, tid, uint32_t(kBlock));
                        for (int s = kWave >> 1; s; s >>= 1) acc += __shfl_xor(acc, s);
                        if ((tid & (kWave - 1)) == 0) part[2][tid >> 6] = acc;
                        __syncthreads();
                        if (tid == 0) {
                            T sum = part[2][0];
                            for (int w = 1; w < kWavesPerBlock; ++w) sum += part[2][w];
                            dst[r] = (identity ? X[P.xoff[j] + r] : T(0)) + sum;
                        }
                        __syncthreads();
                    }
                }
            }
            // words shorter than np - 1: one partial sum per level from this unit's pieces of the levels above np
            for (int k = 1; k < np - 1; ++k) {
                const uint32_t span = P.lv.pw[np - k];
                const uint32_t row = p0 / span, rem = p0 - row * span;
                T acc = T(0);
                for (int j = 1; j <= mt; ++j) {
                    const uint32_t n = P.c * P.lv.pw[j];
                    const T* bseg = other + P.lv.lo[np - k + j] + rem * P.lv.pw[j];
                    const T* xs = X + P.xoff[j];
                    uint32_t z = tid;
                    for (; z + 3 * kBlock < n; z += 4 * kBlock) {      // four loads in flight
                        const T b0 = bseg[z], b1 = bseg[z + kBlock], b2 = bseg[z + 2 * kBlock], b3 = bseg[z + 3 * kBlock];
                        acc = fmadd(xs[z], b0, acc);
                        acc = fmadd(xs[z + kBlock], b1, acc);
                        acc = fmadd(xs[z + 2 * kBlock], b2, acc);
                        acc = fmadd(xs[z + 3 * kBlock], b3, acc);
                    }
                    for (; z < n; z += kBlock) acc = fmadd(xs[z], bseg[z], acc);
                }
                for (int s = kWave >> 1; s; s >>= 1) acc += __shfl_xor(acc, s);
                if ((tid & (kWave - 1)) == 0) part[2][tid >> 6] = acc;
                __syncthreads();
                if (tid == 0) {
                    T sum = part[2][0];
                    for (int w = 1; w < kWavesPerBlock; ++w) sum += part[2][w];
                    dev_add(out + P.lv.lo[k] + row, sum);
                }
                __syncthreads();
            }
        }
    }
}

// ---------------------------------------------------------------------------------------------------------------
// Left factor, d <= 32.  As in chen_adjoint_left_kernel a block owns c words p of length np and copies their pieces of
// the levels np .. N to LDS with coalesced loads (held in registers while the block works on the unit before); the
// top level's copy, and the partial sums of the words shorter than np, are formed from those registers.  The top
// piece (most of the data) is addressed from one wave-uniform base with constant offsets per register; an entry of
// the lower pieces is loaded by the thread that owns it.  The sums inside the block are taken per owner: a thread
// owns one entry q of the pieces 0 .. mt - 1, reads its d children q x from LDS into registers and forms
//   * the whole m = 1 term of dA[q]                                   (B_1: wave-uniform operands),
//   * one partial sum for every ancestor of q inside the block        (B_m from LDS at (q mod d^(m-1)) d + x).
// Numbering the entries of the pieces 0 .. mt end to end, the parent of entry e is (e - c) / d and its children are
// e d + c + x: no per-lane table is needed.  The LDS image gives every run of d children one entry of padding when d
// is even, so that the owners' reads fall into different banks.  Partial sums meet in LDS accumulators (one per
// entry of the pieces 0 .. mt - 1, two sets used in turn); runs of 32 or more lanes that share an ancestor are summed
// in the wave first.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kRowsMaxTop = 8;       // entries of the top piece per thread
constexpr int kRowsMaxLow = 4;       // owned entries per thread

struct RowsPlan {
    int degree, mt, np, upb;
    uint32_t d, c, units, targets, top, bs, pad, img;
    uint32_t eoff[kLeftMaxTile + 2];        // c (d^j - 1) / (d - 1): piece j in the end-to-end numbering
    uint32_t boff[kLeftMaxTile + 2];        // level m of B inside its LDS copy
    uint32_t dmul, dshr;                    // n / d == umulhi(n, dmul) >> dshr for n < 2^31
    StreamLevels lv;
};

template <typename T, int DCEIL, int KT, int KS>
__global__ __launch_bounds__(kBlock) void chen_adjoint_left_rows_kernel(
    const T* __restrict__ dC, T* __restrict__ dA, const T* __restrict__ B, int64_t batch, RowsPlan P, int64_t stride,
    int off, int identity, int64_t dc_share, int64_t dc_stride, int dc_off)
{
    extern __shared__ __align__(16) unsigned char chen_lds[];
    T* Bl = reinterpret_cast<T*>(chen_lds);
    T* Acc = Bl + P.bs;                     // two sets of P.targets accumulators
    T* Img = Acc + 2 * P.targets;           // the unit's pieces 0 .. mt, runs of d children padded
    const uint32_t tid = threadIdx.x, lane = tid & (kWave - 1);
    const int N = P.degree, mt = P.mt, np = P.np;
    const uint32_t d = P.d, c = P.c, dp = d + P.pad;
    const Block2 blk = xcd_block_2d();
    const uint32_t u0 = blk.x * uint32_t(P.upb);
    const uint32_t u1 = u0 + uint32_t(P.upb) < P.units ? u0 + uint32_t(P.upb) : P.units;
    if (u0 >= u1) return;
    // per-thread constants.  Top piece: entry tid + kBlock i and its place in the image.  Owned entry q = tid +
    // kBlock s of the lower pieces: its offset in a row of dC is lgo + p0 * lpw, its place in the image limg.
    uint32_t timg[KT];
#pragma unroll
    for (int i = 0; i < KT; ++i) {
        const uint32_t rel = tid + uint32_t(kBlock) * i;
        const uint32_t x = P.eoff[mt] + rel;
        timg[i] = rel < P.top ? x + P.pad * (__umulhi(x - c, P.dmul) >> P.dshr) : 0xffffffffu;
    }
    uint32_t lgo[KS], lpw[KS], limg[KS];
#pragma unroll
    for (int sl = 0; sl < KS; ++sl) {
        const uint32_t q = tid + uint32_t(kBlock) * sl;
        uint32_t gbt = P.lv.lo[np], pwt = 1;
        for (int jj = 2; jj <= mt; ++jj) {
            const bool in = q >= P.eoff[jj - 1];
            gbt = in ? P.lv.lo[np + jj - 1] - P.eoff[jj - 1] : gbt;
            pwt = in ? P.lv.pw[jj - 1] : pwt;
        }
        lgo[sl] = gbt + q;
        lpw[sl] = q < P.targets ? pwt : 0;      // 0 marks an unused slot
        limg[sl] = q < c ? q : q + P.pad * (__umulhi(q - c, P.dmul) >> P.dshr);
    }
    const uint32_t c1 = np >= 2 ? (P.lv.pw[np] - P.lv.pw[1]) / (d - 1) : 0;      // level shift of the nearest long level
    for (int64_t b = blk.y; b < batch; b += gridDim.y) {
        const T* g = dC + (b / dc_share) * dc_stride + dc_off;
        const T* other = B + b * stride + off;
        T* out = dA + b * stride + off;
        if (off && blk.x == 0 && tid == 0) dA[b * stride] = T(0);
        T rx[KT], rb[KT], rl[KS], rlb[KS];
        auto fetch = [&](uint32_t unit) {
            const uint32_t p0 = unit * c;
            const uint32_t rem1 = np >= 2 ? p0 % P.lv.pw[1] : 0;
            const T* gt = g + P.lv.lo[N] + p0 * P.lv.pw[mt] + tid;
            const T* bt = other + P.lv.lo[1 + mt] + rem1 * P.lv.pw[mt] + tid;
#pragma unroll
            for (int i = 0; i < KT; ++i) {
                const bool ok = timg[i] != 0xffffffffu;
                rx[i] = ok ? gt[kBlock * i] : T(0);
                rb[i] = (ok && np >= 2) ? bt[kBlock * i] : T(0);
            }
#pragma unroll
            for (int sl = 0; sl < KS; ++sl) {
                const bool ok = lpw[sl] != 0;
                rl[sl] = ok ? g[lgo[sl] + p0 * lpw[sl]] : T(0);
                rlb[sl] = (ok && np >= 2 && lpw[sl] > 1) ? other[lgo[sl] + lpw[sl] * (rem1 - c1)] : T(0);
            }
        };
        auto finish = [&](uint32_t unit, T* Aset) {      // stores the complete entries of a unit, clears their sums
            const uint32_t p0 = unit * c;
#pragma unroll
            for (int sl = 0; sl < KS; ++sl) {
                const uint32_t q = tid + uint32_t(kBlock) * sl;
                if (lpw[sl] != 0) {
                    out[lgo[sl] + p0 * lpw[sl]] = Aset[q];
                    Aset[q] = T(0);
                }
            }
        };
        fetch(u0);
        __syncthreads();                                                        // the row before is done with the LDS
        for (uint32_t z = tid; z < P.bs; z += kBlock) Bl[z] = other[z];        // levels 1 .. mt open the row
        for (uint32_t z = tid; z < 2 * P.targets; z += kBlock) Acc[z] = T(0);
        uint32_t flip = 0;
        for (uint32_t unit = u0; unit < u1; ++unit, flip ^= 1) {
            const uint32_t p0 = unit * c;
            T* A = Acc + flip * P.targets;
            __syncthreads();                        // the owners of the unit before have read the image and added their sums
            if (unit > u0) finish(unit - 1, Acc + (flip ^ 1) * P.targets);
            T s1 = T(0);
            {
                T* top = out + P.lv.lo[N] + p0 * P.lv.pw[mt] + tid;            // the top level has no sum
#pragma unroll
                for (int i = 0; i < KT; ++i) {
                    if (timg[i] != 0xffffffffu) {
                        Img[timg[i]] = rx[i];
                        if (identity) top[kBlock * i] = rx[i];
                        s1 = fmadd(rx[i], rb[i], s1);
                    }
                }
#pragma unroll
                for (int sl = 0; sl < KS; ++sl) {
                    if (lpw[sl] != 0) {
                        Img[limg[sl]] = rl[sl];
                        s1 = fmadd(rl[sl], rlb[sl], s1);
                    }
                }
            }
            if (np >= 2) {
                s1 = wave_sum(s1);
                if (lane == 0) dev_add(out + P.lv.lo[np - 1] + p0 / P.lv.pw[1], s1);
            }
            // words shorter than np - 1: their factors are loaded here (deep signatures of few channels)
            for (int k = np - 2; k >= 1; --k) {
                const uint32_t span = P.lv.pw[np - k];
                const uint32_t row = p0 / span, rem = p0 - row * span;
                const uint32_t ck = (P.lv.pw[np] - span) / (d - 1);
                const T* bt = other + P.lv.lo[np - k + mt] + rem * P.lv.pw[mt] + tid;
                T bk[KT], bl[KS];
#pragma unroll
                for (int i = 0; i < KT; ++i) bk[i] = timg[i] != 0xffffffffu ? bt[kBlock * i] : T(0);
#pragma unroll
                for (int sl = 0; sl < KS; ++sl) bl[sl] = lpw[sl] > 1 ? other[lgo[sl] + lpw[sl] * (rem - ck)] : T(0);
                T sk = T(0);
#pragma unroll
                for (int i = 0; i < KT; ++i) sk = fmadd(rx[i], bk[i], sk);
#pragma unroll
                for (int sl = 0; sl < KS; ++sl) sk = fmadd(rl[sl], bl[sl], sk);
                sk = wave_sum(sk);
                if (lane == 0) dev_add(out + P.lv.lo[k] + row, sk);
            }
            __syncthreads();                        // the image is complete
            if (unit + 1 < u1) fetch(unit + 1);
#pragma unroll
            for (int sl = 0; sl < KS; ++sl) {
                const uint32_t q = tid + uint32_t(kBlock) * sl;
                const bool live = lpw[sl] != 0;
                T ch[DCEIL];
                const T* row = Img + c + (live ? q : 0) * dp;
#pragma unroll
                for (int v = 0; v < DCEIL; ++v) ch[v] = (uint32_t(v) < d && live) ? row[v] : T(0);
                T s = (identity && live) ? Img[limg[sl]] : T(0);
#pragma unroll
                for (int v = 0; v < DCEIL; ++v)
                    if (uint32_t(v) < d) s = fmadd(ch[v], other[v], s);       // m = 1: the whole term of q itself
                if (live) lds_add_shared(A + q, s);
                // ancestors inside the block
                uint32_t a = q, rem = 0;
                bool on = live;
                for (int m = 2; m <= mt; ++m) {
                    on = on && a >= c;
                    const uint32_t num = on ? a - c : 0;
                    const uint32_t quo = __umulhi(num, P.dmul) >> P.dshr;
                    rem += (num - quo * d) * P.lv.pw[m - 2];
                    a = quo;
                    T t = T(0);
                    if (on) {
                        const T* br = Bl + P.boff[m] + rem * d;
#pragma unroll
                        for (int v = 0; v < DCEIL; ++v)
                            if (uint32_t(v) < d) t = fmadd(ch[v], br[v], t);
                    }
                    if (P.lv.pw[m - 1] >= 32) {          // long runs of lanes share an ancestor: sum them in the wave
                        uint64_t todo = __ballot(on);
                        while (todo) {
                            const int first = __ffsll((unsigned long long)todo) - 1;
                            const uint32_t key = __shfl(a, first);
                            const bool sel = on && a == key;
                            const T sum = wave_sum(sel ? t : T(0));
                            if (int(lane) == first) lds_add_shared(A + key, sum);
                            todo &= ~__ballot(sel);
                        }
                    } else if (on) {
                        lds_add_shared(A + a, t);
                    }
                }
            }
        }
        __syncthreads();
        finish(u1 - 1, Acc + (flip ^ 1) * P.targets);
    }
}

static inline bool make_rows_plan(RowsPlan& P, uint64_t d, uint64_t degree, uint64_t lds_entries)
{
    if (d < 2 || d > 32 || degree < 2 || !fill_stream_levels(P.lv, d, degree)) return false;
    auto levels = [&](int mt) {      // d + .. + d^mt
        uint64_t s = 0, p = 1;
        for (int j = 1; j <= mt; ++j) { p *= d; s += p; if (s > (uint64_t(1) << 30)) return uint64_t(1) << 30; }
        return s;
    };
    const uint64_t pad = d % 2 == 0 ? 1 : 0;
    // LDS entries: B's levels 1 .. mt, two sets of sums, and the image of c words' pieces with its padding
    auto need = [&](int mt, uint64_t c) {
        const uint64_t targets = c * (levels(mt) + 1 - uint64_t(P.lv.pw[mt]));
        return levels(mt) + 2 * targets + c * (levels(mt) + 1) + pad * targets;
    };
    int mt = 1;
    while (mt + 1 <= int(degree) - 1 && mt + 1 <= kLeftMaxTile && P.lv.pw[mt + 1] != 0 && need(mt + 1, 1) <= lds_entries) ++mt;
    const uint64_t ks_max = d <= 4 ? uint64_t(kRowsMaxLow) : d <= 8 ? 2 : 1;      // owned entries per thread the kernels are built for
    uint64_t c = 0, per = 0;
    for (; mt >= 1 && c == 0; --mt) {
        per = levels(mt) + 1 - uint64_t(P.lv.pw[mt]);      // entries of the pieces 0 .. mt - 1 for c = 1
        double best = 0;
        for (uint64_t cand = 1; cand <= d; ++cand) {
            if (d % cand) continue;
            const uint64_t targets = cand * per, top = cand * uint64_t(P.lv.pw[mt]);
            const uint64_t ks = (targets + kBlock - 1) / kBlock, kt = (top + kBlock - 1) / kBlock;
            if (ks > ks_max || kt > uint64_t(kRowsMaxTop) || need(mt, cand) > lds_entries) continue;
            const double use = 0.3 * double(targets) / double(ks * kBlock) + 0.7 * double(top) / double(kt * kBlock);
            if (use > best + 1e-9) { best = use; c = cand; }
        }
        if (c != 0) break;
    }
    if (c == 0) return false;
    P.degree = int(degree);
    P.mt = mt;
    P.np = int(degree) - mt;
    P.d = uint32_t(d);
    P.c = uint32_t(c);
    P.pad = uint32_t(pad);
    P.units = uint32_t(uint64_t(P.lv.pw[P.np]) / c);
    P.targets = uint32_t(c * per);
    P.top = uint32_t(c * uint64_t(P.lv.pw[mt]));
    P.bs = uint32_t(levels(mt));
    P.img = uint32_t(c * (levels(mt) + 1) + pad * P.targets);
    uint64_t x = 0, p = 1, bo = 0;
    for (int j = 0; j <= mt + 1; ++j) {
        P.eoff[j] = uint32_t(c * x);
        x += p;
        p *= d;
    }
    p = d;
    P.boff[0] = 0;
    for (int m = 1; m <= mt + 1; ++m) {
        P.boff[m] = uint32_t(bo);
        bo += p;
        p *= d;
    }
    const DivBy<uint32_t> dv(d);
    P.dmul = dv.mul;
    P.dshr = dv.shr;
    const uint64_t moved = uint64_t(P.targets) * d;
    P.upb = int(std::max<uint64_t>(1, std::min<uint64_t>((16 * uint64_t(P.bs) + moved - 1) / moved, P.units)));
    return true;
}

static inline bool fill_stream_levels(StreamLevels& lv, uint64_t d, uint64_t degree)
{
    if (degree < 1 || degree > uint64_t(kStreamMaxLevels) || d < 1) return false;
    uint64_t lo = 0, sz = d, pw = 1;
    for (uint64_t t = 0; t <= degree + 1; ++t) {
        lv.pw[t] = pw < (uint64_t(1) << 31) ? uint32_t(pw) : 0u;
        if (t <= degree) pw *= d;
        if (pw >= (uint64_t(1) << 40)) pw = uint64_t(1) << 40;
    }
    for (uint64_t t = 1; t <= degree + 1; ++t) {
        if (lo >= (uint64_t(1) << 31)) return false;
        lv.lo[t] = uint32_t(lo);
        lo += sz;
        if (t <= degree) sz *= d;
        if (sz >= (uint64_t(1) << 40)) sz = uint64_t(1) << 40;
    }
    lv.lo[0] = 0;
    return true;
}

// the lanes' word length: enough words for four waves per row, and a walk of at most kRightMaxRel levels
static inline bool make_right_plan(RightPlan& P, uint64_t d, uint64_t degree)
{
    if (d < 2 || degree < 2 || !fill_stream_levels(P.lv, d, degree)) return false;
    int qmin = 1;
    uint64_t words = d;
    while (words < 256 && qmin < int(degree) - 1) { ++qmin; words *= d; }
    int qe = std::max(qmin, int(degree) - kRightMaxRel);
    if (qe > int(degree) - 1 || qe - 1 > kRightMaxLow) return false;
    P.degree = int(degree);
    P.qe = qe;
    P.rel = int(degree) - qe;
    P.d = uint32_t(d);
    P.words = P.lv.pw[qe];
    return P.words >= 1;
}

// `lds_entries`: LDS entries a block may hold (its pieces of dC plus the low levels of B)
static inline bool make_left_plan(LeftPlan& P, uint64_t d, uint64_t degree, uint64_t lds_entries)
{
    if (d < 2 || degree < 2 || !fill_stream_levels(P.lv, d, degree)) return false;
    auto levels_sum = [&](int mt) {      // 1 + d + .. + d^mt
        uint64_t s = 0, p = 1;
        for (int j = 0; j <= mt; ++j) { s += p; p *= d; if (s > (uint64_t(1) << 30)) return uint64_t(1) << 30; }
        return s;
    };
    auto image = [&](uint64_t c, int mt) {      // LDS entries of a unit: its padded pieces of dC and the levels of B
        uint64_t s = 0, p = 1;
        for (int j = 0; j <= mt; ++j) { s += (c * p + 63) / 64 * 64; p *= d; if (s > (uint64_t(1) << 30)) break; }
        return s + levels_sum(mt);
    };
    int mt = 1;
    while (mt + 1 <= int(degree) - 1 && mt + 1 <= kLeftMaxTile && image(1, mt + 1) <= lds_entries) ++mt;
    if (image(1, mt) > lds_entries) return false;
    uint64_t c = 1;
    for (uint64_t cand = 2; cand <= d; ++cand)
        if (d % cand == 0 && image(cand, mt) <= lds_entries) c = cand;
    P.degree = int(degree);
    P.mt = mt;
    P.np = int(degree) - mt;
    P.d = uint32_t(d);
    P.c = uint32_t(c);
    P.units = uint32_t(uint64_t(P.lv.pw[P.np]) / c);
    uint64_t x = 0, bo = 0, p = 1;
    for (int j = 0; j <= mt + 1; ++j) {        // every piece starts at a multiple of 64 entries
        P.xoff[j] = uint32_t(x);
        x += (c * p + 63) / 64 * 64;
        p *= d;
    }
    P.xs = P.xoff[mt + 1];
    p = d;
    for (int m = 1; m <= mt + 1; ++m) {
        P.boff[m] = uint32_t(bo);
        bo += p;
        p *= d;
    }
    P.boff[0] = 0;
    P.bs = uint32_t(levels_sum(mt) - 1);
    for (int j = 0; j < mt; ++j) {
        const uint64_t rows = c * uint64_t(P.lv.pw[j]);
        uint64_t G = 1;
        while (G * 2 <= 64 && G * 2 * rows <= uint64_t(kBlock) && G < uint64_t(P.lv.pw[mt - j])) G *= 2;
        if (rows <= 3 && P.lv.pw[mt - j] >= uint32_t(kBlock)) G = kBlock;      // the block sums these rows together
        P.gsz[j] = uint32_t(G);
    }
    // the copy of B's levels is shared by the units of a block
    const uint64_t tile = c * uint64_t(P.lv.pw[mt]);
    uint64_t upb = (4 * uint64_t(P.bs) + tile - 1) / tile;
    P.upb = int(std::max<uint64_t>(1, std::min<uint64_t>(upb, P.units)));
    return true;
}

}  // namespace sigamd
