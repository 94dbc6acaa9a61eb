// Reverse signature sweep for paths of many channels (33 and more) at degrees 3 .. 8, where the compiled instance table
// has no faster kernel.
//
// Arithmetic: siglib/cpsig/cp_signature.h:1137-1187 (per step: un-multiply the state by exp(-z), pull the adjoint back
// through the step, emit the increment gradient), regrouped per word as in sig_tree.h with a subtree of depth 1: a
// lane owns a word prefix p of N - 1 letters, the chain S_1[p_1] .. S_{N-1}[p], and the top-level adjoints G[p, a].
//
// What bounds such sweeps is the sum over the prefixes: the gradient of letter a in a step is
//   dz[a] += sum_p G[p, a] * U[p]          (U[p]: Horner value of p towards the top level, one per lane)
// which lanes that each hold one prefix can only form through a reduction across the wave, once per letter and step.
// The top-level adjoints never change during the sweep, so a wave holds its tile of them twice:
//   by prefix:  lane = prefix, registers over the letters:  red[p] = sum_a G[p, a] * z[a] stays inside the lane
//               (z[a] wave-uniform, from scalar loads);
//   by letter:  lane = letter, registers over the prefixes: dz[a] = sum_p G[p, a] * U[p] stays inside the lane too,
//               U[p] handed from lane p to all lanes through LDS.
// No reduction is left but the one over the waves, which the atomic adds into the gradient rows perform.
//
// Tile of a wave: the 64 prefixes (r, 64 blk + lane) that share their first N - 2 letters r, times the KB letters
// [KB ga, KB ga + KB), KB = 64 in single and 32 in double precision (the two copies of the tile take 128 registers
// either way); paths of d channels have ceil(d / 64) values of blk and ceil(d / KB) of ga.  With 32 letters the
// by-letter copy is held by lane = (half h, letter): lanes of half h cover the prefixes 32 h .. 32 h + 31, and the two
// halves' sums meet when the block adds its pieces up.  The first N - 2 prefix letters
// are wave-uniform: their increments come from scalar loads and their gradient pieces need one sum over the wave; the
// last prefix letter differs from lane to lane and its pieces go to the gradient row directly.  The chain and its
// adjoint run through the code of the compiled kernels (Tree / TreeAdj with a one-letter subtree whose adjoint is 1 and
// whose "increment" is red[p]: the pullback then sees exactly the contraction it would have formed itself).
#include <hip/hip_runtime.h>

#include "sig_rows.h"
#include "sig_launch.h"

namespace sigamd {

template <typename T>
constexpr int kRowLettersOf = sizeof(T) == 8 ? 32 : 64;
constexpr int kRowsMinDim = 33;         // below, the compiled table or the other run-time kernels are faster
constexpr int kRowsMinDegree = 3;
constexpr int kRowsMaxDegree = 8;

template <int CTRL>
__device__ __forceinline__ float dpp_moved(float v)
{
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ double dpp_moved(double v)
{
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(v), CTRL, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(v), CTRL, 0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ float lane_value(float v, int l) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l)); }
__device__ __forceinline__ double lane_value(double v, int l)
{
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), l), __builtin_amdgcn_readlane(__double2loint(v), l));
}
// every lane receives the sum over its row of 16 lanes
template <typename T>
__device__ __forceinline__ T row_sum_rows(T v)
{
    v += dpp_moved<0xB1>(v);        // quad_perm [1, 0, 3, 2]
    v += dpp_moved<0x4E>(v);        // quad_perm [2, 3, 0, 1]
    v += dpp_moved<0x141>(v);       // row_half_mirror
    v += dpp_moved<0x140>(v);       // row_mirror
    return v;
}
// sum over the 64 lanes, valid in every lane
template <typename T>
__device__ __forceinline__ T wave_sum_rows(T v)
{
    v = row_sum_rows(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
// lanes 0-31: lo[lane] + lo[lane + 32];  lanes 32-63: hi[lane - 32] + hi[lane]
__device__ __forceinline__ float half_sums(float lo, float hi)
{
    const auto r = __builtin_amdgcn_permlane32_swap(unsigned(__float_as_int(lo)), unsigned(__float_as_int(hi)), false, false);
    return __int_as_float(int(r[0])) + __int_as_float(int(r[1]));
}
__device__ __forceinline__ double half_sums(double lo, double hi) { return pair_sum32(lo, hi); }
// the sums of two values over the 64 lanes for the price of one and a half: the half-waves first exchange halves
template <typename T>
__device__ __forceinline__ void wave_sum_two(T a, T b, T& sum_a, T& sum_b)
{
    const T v = row_sum_rows(half_sums(a, b));
    sum_a = lane_value(v, 0) + lane_value(v, 16);
    sum_b = lane_value(v, 32) + lane_value(v, 48);
}

// Waves per block; a block fills a CU.  Degrees 3 and 4 fit 168 vector registers (three waves per SIMD: 7.0 ms against 7.7 ms
// for 16 paths of 200 steps, 64 channels, degree 4); the longer chains above need more and run two waves per SIMD (a
// third would spill: degree 5 9.4 -> 10.7 ms); double precision always runs two.
template <typename T, int N>
constexpr int kRowsWavesOf = (N <= 4 && sizeof(T) == 4) ? 12 : 8;
constexpr int kRowsMaxWaves = 12;
constexpr int kRowsMaxChunk = 4;                    // steps a block collects before it adds them to the gradient
constexpr int kRowsMaxDim = 4096;                   // a row of the tile per step must leave room for the waves' words
constexpr int kRowsPriv = 2 * kWave;                // a wave's own words per step: by-letter sums, last-prefix-letter pieces (one per lane each)

// both buffers of the row tile and of the waves' own words stay within 64 KB of LDS
inline int rows_chunk_steps(int d, int waves, size_t elem_bytes)
{
    const int c = int(kMaxDynLds / (2 * elem_bytes)) / (d + waves * kRowsPriv);
    return c < 1 ? 1 : c > kRowsMaxChunk ? kRowsMaxChunk : c;
}

template <typename T, int N>
__global__ __launch_bounds__((kRowsWavesOf<T, N> * kWave)) void rows_bwd_kernel(
    const T* __restrict__ inc, const T* __restrict__ sig, const T* __restrict__ gsig,
    T* __restrict__ dzinc, int64_t batch, int64_t L, int d, int64_t sig_stride, int scalar, int64_t rows /* d^(N-2) */,
    int nblk /* ceil(d / 64): blocks of last prefix letters */, int nga /* ceil(d / KB): letter tiles */,
    int64_t blocks_per_path, int chunk /* rows_chunk_steps */)
{
    constexpr int kRowsWaves = kRowsWavesOf<T, N>;
    constexpr int KB = kRowLettersOf<T>;            // letters per tile
    constexpr int HALVES = kWave / KB;              // lane groups of the by-letter copy (1 or 2)
    constexpr int PB = kWave / HALVES;              // prefixes per lane of the by-letter copy
    constexpr int kRowsBlock = kRowsWaves * kWave;
    using Tr = Tree<T, -1, N, 1, 1>;
    using Ad = TreeAdj<T, -1, N, 1, 1>;
    constexpr int M = N - 1;
    static_assert(M >= 2, "degree 3 and up");
    const int lane = threadIdx.x & (kWave - 1);
    const int wib = __builtin_amdgcn_readfirstlane(int(threadIdx.x >> 6));

    // ---- the wave's tile (all wave-uniform) ------------------------------
    // The waves of a block belong to one path: they share the block's gradient tile.  Surplus waves of a path's last
    // block shadow its last tile with all adjoints zero, so that every wave of a block reaches every barrier.
    const int64_t per_path = rows * nblk * nga;
    const int64_t b = int64_t(blockIdx.x) / blocks_per_path;
    int64_t w = (int64_t(blockIdx.x) - b * blocks_per_path) * kRowsWaves + wib;
    const bool valid = w < per_path;
    if (!valid) w = per_path - 1;
    const int ga = int(w % nga);
    w /= nga;
    const int blk = int(w % nblk);
    const int64_t r = w / nblk;
    int pu[M - 1];                          // the shared prefix letters
    {
        int64_t q = r;
#pragma unroll
        for (int l = M - 2; l >= 0; --l) {
            pu[l] = __builtin_amdgcn_readfirstlane(int(q % d));     // wave-uniform: say so (64-bit division is vector code)
            q /= d;
        }
    }
    const int a0 = ga * KB;
    const int last = blk * kWave + lane;      // this lane's last prefix letter
    const bool active = valid && last < d;
    const int lastc = last < d ? last : d - 1;      // idle lanes shadow a valid lane: every load stays in bounds
    const int64_t q = r * d + lastc;

    // ---- state and upstream gradient ------------------------------------
    Tr S;
    Ad A;
    const T* srow = sig + b * sig_stride;
    const T* grow = gsig + b * sig_stride;
    int64_t leaf_off;
    {
        int64_t off = scalar ? 1 : 0, size = d;      // start and size of level l
#pragma unroll
        for (int l = 1; l <= M; ++l) {
            int64_t span = 1;                        // d^(M - l): prefixes of full length below one level-l node
#pragma unroll
            for (int i = l; i < M; ++i) span *= d;
            const int64_t idx = off + q / span;
            // a chain node's adjoint is seeded in one lane only: the recursion is linear in the adjoint
            const bool owner = active && ga == 0 && (q % span == 0);
            S.c[l - 1] = srow[idx];
            A.gc[l - 1] = owner ? grow[idx] : T(0);
            off += size;
            size *= d;
        }
        leaf_off = off;
    }
    // by prefix: this lane's prefix, the tile's letters
    T gp[KB];
    {
        const T* g = grow + leaf_off + q * d + a0;
#pragma unroll
        for (int a = 0; a < KB; ++a) {
            const bool ok = active && a0 + a < d;
            const T v = g[ok ? a : 0];
            gp[a] = ok ? v : T(0);
        }
    }
    A.gs[0] = T(1);
    S.s[0] = T(0);
    // by letter: this lane's letter, the tile's prefixes
    const int my_letter = a0 + (lane & (KB - 1));
    const int my_half = lane / KB;                  // prefixes PB * my_half .. of the tile
    const bool letter_ok = my_letter < d;
    T gt[PB];
    {
        const bool lok = valid && letter_ok;
        const int p0 = blk * kWave + my_half * PB;  // first of this lane's prefixes (as last prefix letter)
        // (a half that lies wholly beyond the row reads, and drops, the row's last prefix: every load stays in bounds)
        const T* g = grow + leaf_off + (r * d + (p0 < d ? p0 : d - 1)) * d + (lok ? my_letter : 0);
#pragma unroll
        for (int j = 0; j < PB; ++j) {
            const bool ok = lok && p0 + j < d;
            const T v = g[ok ? int64_t(j) * d : 0];
            gt[j] = ok ? v : T(0);
        }
    }

    // ---- the sweep ---------------------------------------------------------
    // Increments are [batch][L + 2][d] with a zero row at either end of a path.  The tile's slice of a step's row is
    // wave-uniform and arrives through scalar loads, requested one step ahead; a slice that reaches past the row reads
    // on into the next row of the same path (fewer elements than a row holds) and meets adjoints that are zero.  The
    // Horner values U[p] go from the by-prefix lanes to the by-letter lanes through the wave's LDS slot: one write, then
    // every lane reads all of it (same address in every lane: a broadcast).
    //
    // Gradient pieces of a step: the by-letter sums and the pieces of the last prefix letter (one per lane each) go to
    // words of the wave's own in LDS with plain writes (a float LDS atomic of a full wave costs about 500 cycles here);
    // the few pieces of the shared prefix letters are added to the block's row tile with LDS atomics.  After `chunk`
    // steps the whole block sums, per step and letter, the tile and the words of the waves that cover the letter, adds
    // the sum to the gradient row and clears the tile, while the waves already fill the other buffer: one barrier per
    // chunk.
    extern __shared__ double rows_lds_raw[];
    T* rows_lds = reinterpret_cast<T*>(rows_lds_raw);
    __shared__ __attribute__((aligned(16))) T ul_all[kRowsWaves][kWave];
    __shared__ int wave_a0[kRowsWaves], wave_l0[kRowsWaves];
    T* ul = ul_all[wib];
    const int tile_elems = chunk * d;                               // per buffer
    const int priv_elems = chunk * kRowsWaves * kRowsPriv;          // per buffer
    T* tile = rows_lds;                                             // [2][chunk][d]
    T* priv = rows_lds + 2 * tile_elems;                            // [2][chunk][wave][kRowsPriv]
    for (int e = threadIdx.x; e < 2 * tile_elems; e += kRowsBlock) tile[e] = T(0);
    if (lane == 0) {
        wave_a0[wib] = a0;
        wave_l0[wib] = blk * kWave;
    }
    __syncthreads();

    const T* zrow = inc + (b * (L + 2) + L) * d;        // row of the last step
    typename Tr::Inc in;
    in.z[0] = T(0);
    T zs[KB];
    T pz_next[M];
    auto fetch = [&](const T* row) {
#pragma unroll
        for (int l = 0; l < M - 1; ++l) pz_next[l] = row[pu[l]];
        pz_next[M - 1] = row[lastc];
#pragma unroll
        for (int a = 0; a < KB; ++a) zs[a] = row[a0 + a];
    };
    fetch(zrow);
    int buf = 0, sidx = 0;
    int64_t t_first = L - 1;                // step held by row 0 of the current buffer
    for (int64_t t = L - 1; t >= 0; --t) {
#pragma unroll
        for (int l = 0; l < M; ++l) in.pz[l] = pz_next[l];

        // state before the step, and the prefix's Horner value towards the top level: it does not depend on the
        // adjoints, so it is on its way through LDS while the contraction with the letters runs
        typename Tr::Chain unmul;
        S.template fwd_step<AllLetters, true>(in, &unmul);
        if constexpr (Tr::kLockstep) {
            typename Tr::Chain ch;
            S.template chain_all<false>(in, ch, &unmul);
            ul[lane] = ch.u[N][M - 1];
        } else {
            T u[M];
            S.template chain_u<N, M>(in, u);
            ul[lane] = u[M - 1];
        }
        __builtin_amdgcn_sched_barrier(0);

        // by prefix: red = sum over the tile's letters of G[p, a] * z[a]
        T red0 = T(0), red1 = T(0);
#pragma unroll
        for (int a = 0; a < KB; a += 2) {
            red0 = fmadd(gp[a], zs[a], red0);
            red1 = fmadd(gp[a + 1], zs[a + 1], red1);
        }
        in.zs[0] = red0 + red1;
        __builtin_amdgcn_sched_barrier(0);
        // the step before this one (step 0 fetches the zero row in front of the path)
        zrow -= d;
        fetch(zrow);
        __builtin_amdgcn_sched_barrier(0);

        typename Ad::DInc dz;
        dz.dj[0] = T(0);
        dz.da[0] = T(0);
#pragma unroll
        for (int l = 0; l < M; ++l) dz.dc[l] = T(0);
        A.template pullback<-1, AllLetters>(S, in, dz, Tr::kLockstep ? &unmul : nullptr);

        // the shared prefix letters: one sum over the wave each
        T mine = T(0);
        int where = 0;
#pragma unroll
        for (int l = 0; l + 1 < M - 1; l += 2) {
            T s0, s1;
            wave_sum_two(dz.dc[l], dz.dc[l + 1], s0, s1);
            if (lane == l) {
                mine = s0;
                where = pu[l];
            }
            if (lane == l + 1) {
                mine = s1;
                where = pu[l + 1];
            }
        }
        if constexpr ((M - 1) & 1) {
            const T s = wave_sum_rows(dz.dc[M - 2]);
            if (lane == M - 2) {
                mine = s;
                where = pu[M - 2];
            }
        }
        if (lane < M - 1) lds_add_shared(&tile[(buf * chunk + sidx) * d + where], mine);

        // by letter: dz[a] = sum over this lane's prefixes of G[p, a] * U[p]
        T acc0 = T(0), acc1 = T(0);
        constexpr int V = int(16 / sizeof(T));                  // values per 16-byte LDS read
        struct alignas(16) Vec { T v[V]; };
        const Vec* us = reinterpret_cast<const Vec*>(ul + my_half * PB);
#pragma unroll
        for (int jb = 0; jb < PB; jb += 16) {
            Vec v[16 / V];
#pragma unroll
            for (int i = 0; i < 16 / V; ++i) v[i] = us[jb / V + i];
#pragma unroll
            for (int i = 0; i < 16; i += 2) {
                acc0 = fmadd(gt[jb + i], v[i / V].v[i % V], acc0);
                acc1 = fmadd(gt[jb + i + 1], v[(i + 1) / V].v[(i + 1) % V], acc1);
            }
            __builtin_amdgcn_sched_barrier(0);      // sixteen values in flight at a time: registers
        }
        // idle lanes and shadow waves hold zero adjoints: what they write is zero
        T* mine_row = priv + ((buf * chunk + sidx) * kRowsWaves + wib) * kRowsPriv;
        mine_row[lane] = acc0 + acc1;
        mine_row[kWave + lane] = dz.dc[M - 1];

        if (++sidx == chunk || t == 0) {
            __syncthreads();
            // rows 0 .. sidx - 1 of the buffer hold the steps t_first, t_first - 1, ..
            T* src = tile + buf * tile_elems;
            const T* pr = priv + buf * priv_elems;
            T* out = dzinc + (b * L + t_first) * d;
            for (int e = threadIdx.x; e < sidx * d; e += kRowsBlock) {
                const int row = e / d, a = e - row * d;
                T v = src[e];
                src[e] = T(0);
#pragma unroll 1
                for (int k = 0; k < kRowsWaves; ++k) {
                    const T* wr = pr + (row * kRowsWaves + k) * kRowsPriv;
                    const unsigned ia = unsigned(a - wave_a0[k]), il = unsigned(a - wave_l0[k]);
                    if (ia < unsigned(KB)) {
                        v += wr[ia];
                        if constexpr (HALVES == 2) v += wr[KB + ia];
                    }
                    if (il < unsigned(kWave)) v += wr[kWave + il];
                }
                dev_add(&out[a - int64_t(row) * d], v);      // row `row` lies `row` gradient rows before t_first
            }
            t_first -= sidx;
            sidx = 0;
            buf ^= 1;
        }
    }
}

// ---------------------------------------------------------------------------
// Forward sweep in the same tiling (arithmetic: siglib/cpsig/cp_signature.h:464-499): a lane owns the prefix
// (r, 64 blk + lane), its chain, and the KB top-level coefficients (prefix, letter) of the wave's letter tile.  Per step
// the top level costs one multiply-add per coefficient, S_N[p, a] += U[p] * z[a], with z[a] wave-uniform from scalar
// loads; the chain work of a lane is shared by 64 (32) of them instead of the 16 or 32 of the general run-time kernels.
// The letters are held in two halves: the next step's half is requested as soon as this step is done with it, so a
// row never sits in the scalar registers twice.
// ---------------------------------------------------------------------------
template <typename T, int N>
__global__ __launch_bounds__(kBlock) void rows_fwd_kernel(
    const T* __restrict__ inc, T* __restrict__ out, int64_t batch, int64_t L, int d, int64_t out_stride, int scalar,
    int64_t rows /* d^(N-2) */, int nblk, int nga, int* __restrict__ nonfinite)
{
    constexpr int KB = kRowLettersOf<T>;
    constexpr int HB = KB / 2;
    using Tr = Tree<T, -1, N, 1, 1>;
    constexpr int M = N - 1;
    static_assert(M >= 2, "degree 3 and up");
    const int lane = threadIdx.x & (kWave - 1);
    int64_t wave = int64_t(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
    {
        const uint32_t wlo = __builtin_amdgcn_readfirstlane(uint32_t(wave));
        const uint32_t whi = __builtin_amdgcn_readfirstlane(uint32_t(uint64_t(wave) >> 32));
        wave = int64_t((uint64_t(whi) << 32) | wlo);
    }
    const int64_t per_path = rows * nblk * nga;
    const int64_t b = wave / per_path;
    if (b >= batch) return;
    int64_t w = wave - b * per_path;
    const int ga = int(w % nga);
    w /= nga;
    const int blk = int(w % nblk);
    const int64_t r = w / nblk;
    int pu[M - 1];                          // the shared prefix letters
    {
        int64_t q = r;
#pragma unroll
        for (int l = M - 2; l >= 0; --l) {
            pu[l] = __builtin_amdgcn_readfirstlane(int(q % d));     // wave-uniform: say so (64-bit division is vector code)
            q /= d;
        }
    }
    const int a0 = ga * KB;
    const int last = blk * kWave + lane;
    const bool active = last < d;
    const int lastc = active ? last : d - 1;        // idle lanes shadow a valid lane: every load stays in bounds
    const int64_t q = r * d + lastc;

    Tr S;
#pragma unroll
    for (int l = 0; l < M; ++l) S.c[l] = T(0);
    S.s[0] = T(0);
    T leaf[KB];
#pragma unroll
    for (int a = 0; a < KB; ++a) leaf[a] = T(0);

    // increments [batch][L + 2][d] with a zero row at either end of a path; a letter tile that reaches past the row reads
    // on into the next row of the same path (fewer elements than a row holds): those coefficients are never stored
    const T* zrow = inc + (b * (L + 2) + 1) * d;        // row of the first step
    typename Tr::Inc in;
    in.z[0] = T(0);
    in.zs[0] = T(0);
    T za[HB], zb[HB], pz_next[M];
    auto fetch_prefix = [&](const T* row) {
#pragma unroll
        for (int l = 0; l < M - 1; ++l) pz_next[l] = row[pu[l]];
        pz_next[M - 1] = row[lastc];
    };
    fetch_prefix(zrow);
#pragma unroll
    for (int a = 0; a < HB; ++a) za[a] = zrow[a0 + a];
#pragma unroll
    for (int a = 0; a < HB; ++a) zb[a] = zrow[a0 + HB + a];
    for (int64_t t = 0; t < L; ++t) {
#pragma unroll
        for (int l = 0; l < M; ++l) in.pz[l] = pz_next[l];
        zrow += d;                                      // after the last step: the zero row behind the path
        fetch_prefix(zrow);
        // the prefix's Horner value towards the top level, from the state before the step
        T u;
        if constexpr (Tr::kLockstep) {
            typename Tr::Chain ch;
            S.fwd_step(in, &ch);
            u = ch.u[N][M - 1];
        } else {
            T uu[M];
            S.template chain_u<N, M>(in, uu);
            u = uu[M - 1];
            S.fwd_step(in);
        }
#pragma unroll
        for (int a = 0; a < HB; ++a) leaf[a] = fmadd(u, za[a], leaf[a]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < HB; ++a) za[a] = zrow[a0 + a];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < HB; ++a) leaf[HB + a] = fmadd(u, zb[a], leaf[HB + a]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int a = 0; a < HB; ++a) zb[a] = zrow[a0 + HB + a];
        __builtin_amdgcn_sched_barrier(0);
    }

    if (!active) return;
    T* o = out + b * out_stride;
    if (scalar && r == 0 && blk == 0 && ga == 0 && lane == 0) o[0] = T(1);
    // chk stays 0 while every stored value is finite: x * 0 is NaN for x = NaN or +-Inf
    T chk = T(0);
    int64_t off = scalar ? 1 : 0, size = d;
#pragma unroll
    for (int l = 1; l <= M; ++l) {
        int64_t span = 1;                            // d^(M - l): prefixes of full length below one level-l node
#pragma unroll
        for (int i = l; i < M; ++i) span *= d;
        // a chain node is stored by the lane whose remaining prefix letters are 0, in the first letter tile
        if (ga == 0 && q % span == 0) {
            o[off + q / span] = S.c[l - 1];
            chk = fmadd(S.c[l - 1], T(0), chk);
        }
        off += size;
        size *= d;
    }
    T* top = o + off + q * d + a0;
#pragma unroll
    for (int a = 0; a < KB; ++a) {
        if (a0 + a < d) {
            top[a] = leaf[a];
            chk = fmadd(leaf[a], T(0), chk);
        }
    }
    if (nonfinite && !(chk == T(0))) *nonfinite = 1;
}

template <typename T, int N>
hipError_t launch_rows_fwd_n(const FwdParams& p)
{
    const int nblk = (p.d + kWave - 1) / kWave, nga = (p.d + kRowLettersOf<T> - 1) / kRowLettersOf<T>;
    int64_t rows = 1;
    for (int i = 0; i < N - 2; ++i) rows *= p.d;
    const int64_t waves = p.batch * rows * nblk * nga;
    const int64_t blocks = (waves + kWavesPerBlock - 1) / kWavesPerBlock;
    if (blocks < 1 || blocks > kMaxGridX) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((rows_fwd_kernel<T, N>), dim3(unsigned(blocks)), dim3(kBlock), 0, p.stream, static_cast<const T*>(p.inc),
                       static_cast<T*>(p.out), p.batch, p.L, p.d, p.out_stride, p.scalar, rows, nblk, nga, p.nonfinite);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_rows_fwd(const FwdParams& p, int degree)
{
    if (p.nseg != 1 || p.from_points || p.d < kRowsMinDim || p.d > kRowsMaxDim) return hipErrorInvalidConfiguration;
    switch (degree) {
        case 3: return launch_rows_fwd_n<T, 3>(p);
        case 4: return launch_rows_fwd_n<T, 4>(p);
        case 5: return launch_rows_fwd_n<T, 5>(p);
        case 6: return launch_rows_fwd_n<T, 6>(p);
        case 7: return launch_rows_fwd_n<T, 7>(p);
        case 8:
            if constexpr (sizeof(T) == 4) return launch_rows_fwd_n<T, 8>(p);
            return hipErrorInvalidConfiguration;
        default: return hipErrorInvalidConfiguration;
    }
}
template hipError_t launch_rows_fwd<float>(const FwdParams&, int);
template hipError_t launch_rows_fwd<double>(const FwdParams&, int);

template <typename T, int N>
hipError_t launch_rows(const BwdParams& p)
{
    constexpr int kRowsWaves = kRowsWavesOf<T, N>;
    const int nblk = (p.d + kWave - 1) / kWave, nga = (p.d + kRowLettersOf<T> - 1) / kRowLettersOf<T>;
    int64_t rows = 1;
    for (int i = 0; i < N - 2; ++i) rows *= p.d;
    const int64_t per_path = rows * nblk * nga;
    const int64_t blocks_per_path = (per_path + kRowsWaves - 1) / kRowsWaves;
    const int64_t blocks = p.batch * blocks_per_path;
    if (blocks < 1 || blocks > kMaxGridX) return hipErrorInvalidConfiguration;
    const int chunk = rows_chunk_steps(p.d, kRowsWaves, sizeof(T));
    const size_t lds = size_t(2) * chunk * (size_t(p.d) + kRowsWaves * kRowsPriv) * sizeof(T);
    if (lds > kMaxDynLds) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL((rows_bwd_kernel<T, N>), dim3(unsigned(blocks)), dim3(kRowsWaves * kWave), lds, p.stream,
                       static_cast<const T*>(p.inc), static_cast<const T*>(p.sig), static_cast<const T*>(p.gsig),
                       static_cast<T*>(p.dzinc), p.batch, p.L, p.d, p.sig_stride, p.scalar, rows, nblk, nga, blocks_per_path, chunk);
    return hipGetLastError();
}

bool rows_bwd_supported(size_t elem_bytes, uint64_t d, uint64_t degree)
{
    if (elem_bytes == 8 && degree > 7) return false;     // (its 56 chain values per lane no longer fit the registers)
    return (elem_bytes == 4 || elem_bytes == 8) && d >= uint64_t(kRowsMinDim) && d <= uint64_t(kRowsMaxDim) && degree >= uint64_t(kRowsMinDegree) &&
           degree <= uint64_t(kRowsMaxDegree);
}

bool rows_bwd_fits(size_t elem_bytes, uint64_t d, uint64_t degree, uint64_t batch)
{
    const uint64_t nblk = (d + kWave - 1) / kWave, nga = elem_bytes == 8 ? (d + 31) / 32 : nblk;
    unsigned __int128 per_path = (unsigned __int128)nblk * nga;
    for (uint64_t i = 0; i + 2 < degree; ++i) {
        per_path *= d;
        if (per_path > (unsigned __int128)kMaxGridX * 8) return false;
    }
    const unsigned __int128 blocks = (per_path + 7) / 8 * batch;      // at the smaller of the two block sizes
    return blocks >= 1 && blocks <= (unsigned __int128)kMaxGridX;
}

template <typename T>
hipError_t launch_rows_bwd(const BwdParams& p, int degree)
{
    if (p.nseg != 1 || p.from_points || p.d < kRowsMinDim || p.d > kRowsMaxDim) return hipErrorInvalidConfiguration;
    switch (degree) {
        case 3: return launch_rows<T, 3>(p);
        case 4: return launch_rows<T, 4>(p);
        case 5: return launch_rows<T, 5>(p);
        case 6: return launch_rows<T, 6>(p);
        case 7: return launch_rows<T, 7>(p);
        case 8:
            if constexpr (sizeof(T) == 4) return launch_rows<T, 8>(p);
            return hipErrorInvalidConfiguration;
        default: return hipErrorInvalidConfiguration;
    }
}
template hipError_t launch_rows_bwd<float>(const BwdParams&, int);
template hipError_t launch_rows_bwd<double>(const BwdParams&, int);

}  // namespace sigamd
