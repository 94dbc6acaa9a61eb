// Signature sweeps of run-time degree, for degrees beyond the compiled instance table (17 .. 64).
//
// Counterpart of the reference's run-time-degree kernels (siglib/cusig/cu_signature.cu:396-491 forward,
// :497-919 backward, limit :3022-3025).  A signature of degree >= 17 only fits in memory for 2, 3 or 4 (augmented)
// channels, so the dimension is a compile-time constant D in {2, 3, 4}.
//
// Partition: as in the compiled tree kernels a lane owns a word prefix p of length M = N - TAIL, the chain
// S_1[p_1] .. S_M[p] and the whole subtree of depth TAIL below p.  The subtree lives in registers and is walked by
// the same code as in the compiled kernels (Tree::fwd_desc / TreeAdj::bwd_desc); the chain has run-time length and
// lives in LDS, one column per lane (row stride 64 words: conflict-free), next to the step's increments gathered
// along the prefix.  Arithmetic: siglib/cpsig/cp_signature.h:464-499 (forward), :1137-1187 (backward), regrouped
// per word exactly as in sig_tree.h.
#include <hip/hip_runtime.h>

#include "sig_deep.h"
#include "sig_launch.h"

namespace sigamd {

// depth of the register-resident subtree per dimension (values per lane: D = 2: 30, D = 3: 39, D = 4: 20)
template <int D>
struct DeepTail {
    static constexpr int value = D == 2 ? 4 : D == 3 ? 3 : 2;
};

constexpr int kDeepLanes = 64;      // one wave per block: the LDS columns of a block belong to one wave

template <typename T, int D>
struct Deep {
    static constexpr int TAIL = DeepTail<D>::value;
    using Sub = Tree<T, D, TAIL + 1, TAIL, D>;       // only its subtree part is used
    using Adj = TreeAdj<T, D, TAIL + 1, TAIL, D>;
    using Inc = typename Sub::Inc;

    int M, N;
    T* c;           // chain: c[l * 64] = S_{l+1}[p_1 .. p_{l+1}]
    T* pz;          // pz[l * 64] = z[p_{l+1}] of the current step
    const T* rtab;  // rtab[k] = 1 / k
    uint64_t lo, hi;    // the prefix letters, two bits each (letter l at bit 2 l)
    Sub S;

    __device__ __forceinline__ int letter(int l) const { return int(((l < 32) ? (lo >> (2 * l)) : (hi >> (2 * (l - 32)))) & 3u); }

    __device__ __forceinline__ void set_prefix(int64_t q)
    {
        lo = hi = 0;
        for (int l = M - 1; l >= 0; --l) {
            const uint64_t digit = uint64_t(q % D);
            q /= D;
            if (l < 32) lo |= digit << (2 * l);
            else hi |= digit << (2 * (l - 32));
        }
    }

    static __device__ __forceinline__ T pick(const T (&z)[D], int a)
    {
        T v = z[0];
#pragma unroll
        for (int j = 1; j < D; ++j) v = (a == j) ? z[j] : v;
        return v;
    }

    // gathers the step's increments along the prefix and fills the letters of the subtree
    __device__ __forceinline__ void load_step(const T* __restrict__ row, Inc& in)
    {
        T z[D];
#pragma unroll
        for (int j = 0; j < D; ++j) z[j] = row[j];
#pragma unroll
        for (int j = 0; j < D; ++j) { in.z[j] = z[j]; in.zs[j] = z[j]; }
        in.pz[0] = T(0);
        for (int l = 0; l < M; ++l) pz[l * kDeepLanes] = pick(z, letter(l));
    }

    // S <- S (x) exp(SIGN * z), target levels descending (every read of a lower level sees the value from before
    // the step); `in` holds SIGN * z for the subtree
    template <int SIGN>
    __device__ __forceinline__ void fwd_step(const Inc& in)
    {
        const T sg = T(SIGN);
        for (int t = N; t >= 2; --t) {
            const int depth = t - 1 < M ? t - 1 : M;
            T u = fmadd(sg * pz[0], rtab[t], c[0]);
            for (int l = 1; l < depth; ++l) u = fmadd(u * rtab[t - l], sg * pz[l * kDeepLanes], c[l * kDeepLanes]);
            if (t <= M) {
                c[(t - 1) * kDeepLanes] = fmadd(u, sg * pz[(t - 1) * kDeepLanes], c[(t - 1) * kDeepLanes]);
            } else {
                static_for<1, TAIL>([&](auto ic) {
                    constexpr int I = decltype(ic)::value;
                    if (t - M == I) S.template fwd_desc<1, I>(in, u, 0);
                });
            }
        }
        c[0] += sg * pz[0];
    }
};

template <typename T>
__device__ __forceinline__ void fill_recip(T* rtab, int n, int lane)
{
    for (int k = lane; k <= n; k += kDeepLanes) rtab[k] = k ? T(1) / T(k) : T(0);
}

// inc: [batch][L + 2][D] with a zero row at either end of every path; out: [batch][out_stride]
template <typename T, int D>
__global__ __launch_bounds__(kDeepLanes) void deep_fwd_kernel(
    const T* __restrict__ inc, T* __restrict__ out, int64_t batch, int64_t L, int N, int64_t out_stride, int scalar,
    int64_t P, int64_t wpp, int* __restrict__ nonfinite)
{
    using Dp = Deep<T, D>;
    using Sub = typename Dp::Sub;
    constexpr int TAIL = Dp::TAIL;
    extern __shared__ double deep_lds_raw[];
    T* lds = reinterpret_cast<T*>(deep_lds_raw);
    const int lane = threadIdx.x;
    Dp dp;
    dp.N = N;
    dp.M = N - TAIL;
    const int M = dp.M;
    dp.c = lds + lane;
    dp.pz = lds + int64_t(M) * kDeepLanes + lane;
    T* rtab = lds + 2 * int64_t(M) * kDeepLanes;
    fill_recip(rtab, N, lane);
    dp.rtab = rtab;

    // one wave serves 64 consecutive prefixes of one path (wpp waves per path; the last may be partly idle)
    const int64_t b = int64_t(blockIdx.x) / wpp;
    int64_t q = (int64_t(blockIdx.x) % wpp) * kDeepLanes + lane;
    const bool active = q < P;
    if (!active) q = P - 1;             // idle lanes shadow a valid one and never store
    dp.set_prefix(q);
    for (int l = 0; l < M; ++l) dp.c[l * kDeepLanes] = T(0);
#pragma unroll
    for (int i = 0; i < Sub::SUB; ++i) dp.S.s[i] = T(0);
    __syncthreads();                    // the reciprocal table is complete

    const T* row = inc + (b * (L + 2) + 1) * D;
    for (int64_t t = 0; t < L; ++t) {
        typename Dp::Inc in;
        dp.load_step(row, in);
        dp.template fwd_step<1>(in);
        row += D;
    }

    if (!active) return;
    T* o = out + b * out_stride;
    if (scalar && q == 0) o[0] = T(1);
    T chk = T(0);
    {
        // chain nodes are stored by the lane whose remaining prefix letters are 0
        int64_t rest = 1;               // D^(M - l)
        int64_t lo_l = (scalar ? 1 : 0);
        // offsets of levels 1 .. M
        int64_t off[kDeepMaxDegree + 1];
        int64_t sz = D;
        for (int l = 1; l <= N; ++l) { off[l] = lo_l; lo_l += sz; sz *= D; }
        for (int l = M; l >= 1; --l) {
            const T v = dp.c[(l - 1) * kDeepLanes];
            if (q % rest == 0) o[off[l] + q / rest] = v;
            chk = fmadd(v, T(0), chk);
            rest *= D;
        }
        static_for<1, TAIL>([&](auto ec) {
            constexpr int e = decltype(ec)::value;
            constexpr int cnt = int(ipow64(D, e));      // subtree values at depth e
            const int64_t base = off[M + e] + q * cnt;
#pragma unroll
            for (int r = 0; r < cnt; ++r) o[base + r] = dp.S.s[Sub::off(e) + r];
        });
    }
#pragma unroll
    for (int i = 0; i < Sub::SUB; ++i) chk = fmadd(dp.S.s[i], T(0), chk);
    if (nonfinite && !(chk == T(0))) *nonfinite = 1;
}

// Reverse sweep: per step un-multiply the state by exp(-z), pull the adjoint back through the step (target levels
// ascending), sum the wave's increment-gradient pieces and add them to dz[path][step][letter].
template <typename T, int D>
__global__ __launch_bounds__(kDeepLanes) void deep_bwd_kernel(
    const T* __restrict__ inc, const T* __restrict__ sig, const T* __restrict__ gsig, T* __restrict__ dzinc,
    int64_t batch, int64_t L, int N, int64_t sig_stride, int scalar, int64_t P, int64_t wpp)
{
    using Dp = Deep<T, D>;
    using Sub = typename Dp::Sub;
    using Adj = typename Dp::Adj;
    constexpr int TAIL = Dp::TAIL;
    extern __shared__ double deep_lds_raw[];
    T* lds = reinterpret_cast<T*>(deep_lds_raw);
    const int lane = threadIdx.x;
    Dp dp;
    dp.N = N;
    dp.M = N - TAIL;
    const int M = dp.M;
    dp.c = lds + lane;
    dp.pz = lds + int64_t(M) * kDeepLanes + lane;
    T* gc = lds + 2 * int64_t(M) * kDeepLanes + lane;       // partial adjoints of the chain nodes
    T* uc = lds + 3 * int64_t(M) * kDeepLanes + lane;       // Horner values along the prefix of the level at hand
    T* rtab = lds + 4 * int64_t(M) * kDeepLanes;
    fill_recip(rtab, N, lane);
    dp.rtab = rtab;

    const int64_t b = int64_t(blockIdx.x) / wpp;
    int64_t q = (int64_t(blockIdx.x) % wpp) * kDeepLanes + lane;
    const bool active = q < P;
    if (!active) q = P - 1;
    dp.set_prefix(q);

    // ---- state and upstream gradient ----
    Adj A;
    const T* srow = sig + b * sig_stride;
    const T* grow = gsig + b * sig_stride;
    {
        int64_t off[kDeepMaxDegree + 1];
        int64_t lo_l = (scalar ? 1 : 0), sz = D;
        for (int l = 1; l <= N; ++l) { off[l] = lo_l; lo_l += sz; sz *= D; }
        int64_t rest = 1;
        for (int l = M; l >= 1; --l) {
            const int64_t idx = off[l] + q / rest;
            dp.c[(l - 1) * kDeepLanes] = srow[idx];
            // the adjoint of a shared chain node is seeded in one lane only: the recursion is linear in the adjoint
            gc[(l - 1) * kDeepLanes] = (active && q % rest == 0) ? grow[idx] : T(0);
            rest *= D;
        }
        static_for<1, TAIL>([&](auto ec) {
            constexpr int e = decltype(ec)::value;
            constexpr int cnt = int(ipow64(D, e));
            const int64_t base = off[M + e] + q * cnt;
#pragma unroll
            for (int r = 0; r < cnt; ++r) {
                dp.S.s[Sub::off(e) + r] = srow[base + r];
                A.gs[Sub::off(e) + r] = active ? grow[base + r] : T(0);
            }
        });
    }
    A.gc[0] = T(0);
    __syncthreads();

    const T* row = inc + (b * (L + 2) + L) * D;          // row of the last step
    for (int64_t t = L - 1; t >= 0; --t) {
        typename Dp::Inc in, neg;
        dp.load_step(row, in);
#pragma unroll
        for (int j = 0; j < D; ++j) { neg.z[j] = -in.z[j]; neg.zs[j] = -in.zs[j]; }
        neg.pz[0] = T(0);
        dp.template fwd_step<-1>(neg);                   // state before the step

        T dj[D];
#pragma unroll
        for (int j = 0; j < D; ++j) dj[j] = T(0);
        auto add_letter = [&](int a, T v) {
#pragma unroll
            for (int j = 0; j < D; ++j) dj[j] += (a == j) ? v : T(0);
        };
        add_letter(dp.letter(0), gc[0]);                 // level 1
        for (int lev = 2; lev <= N; ++lev) {
            const int depth = lev - 1 < M ? lev - 1 : M;
            T u = fmadd(dp.pz[0], rtab[lev], dp.c[0]);
            uc[0] = u;
            for (int l = 1; l < depth; ++l) {
                u = fmadd(u * rtab[lev - l], dp.pz[l * kDeepLanes], dp.c[l * kDeepLanes]);
                uc[l * kDeepLanes] = u;
            }
            T adj;
            int from;
            if (lev <= M) {
                adj = gc[(lev - 1) * kDeepLanes];
                from = lev;
            } else {
                typename Adj::DInc dz;
#pragma unroll
                for (int j = 0; j < D; ++j) { dz.dj[j] = T(0); dz.da[j] = T(0); }
                dz.dc[0] = T(0);
                T red = T(0);
                static_for<1, TAIL>([&](auto ic) {
                    constexpr int I = decltype(ic)::value;
                    if (lev - M == I) red = A.template bwd_desc<1, I, 0>(dp.S, in, dz, u, 0);
                });
#pragma unroll
                for (int j = 0; j < D; ++j) dj[j] += dz.dj[j];
                gc[(M - 1) * kDeepLanes] += red;
                adj = red;
                from = M;
            }
            // walk the adjoint of chain node `from` up to the root
            for (int l = from - 1; l >= 1; --l) {
                const T sc = rtab[lev - l];
                const T v = uc[(l - 1) * kDeepLanes] * sc;
                add_letter(dp.letter(l), adj * v);
                adj = adj * dp.pz[l * kDeepLanes] * sc;
                gc[(l - 1) * kDeepLanes] += adj;
            }
            add_letter(dp.letter(0), adj * rtab[lev]);
        }

        // idle lanes carry zero adjoints, so their pieces are zero
#pragma unroll
        for (int j = 0; j < D; ++j) {
            T v = dj[j];
            for (int o = kDeepLanes / 2; o >= 1; o >>= 1) v += __shfl_xor(v, o);
            if (lane == 0) dev_add(&dzinc[(b * L + t) * D + j], v);
        }
        row -= D;
    }
}

bool deep_supported(uint64_t d, uint64_t degree)
{
    const uint64_t tail = d == 2 ? DeepTail<2>::value : d == 3 ? DeepTail<3>::value : DeepTail<4>::value;
    return d >= 2 && d <= 4 && degree >= tail + 1 && degree <= uint64_t(kDeepMaxDegree);
}

bool deep_fits(uint64_t d, uint64_t degree, uint64_t batch)
{
    if (!deep_supported(d, degree) || batch < 1) return false;
    const uint64_t tail = d == 2 ? DeepTail<2>::value : d == 3 ? DeepTail<3>::value : DeepTail<4>::value;
    uint64_t prefixes = 1;
    for (uint64_t l = 0; l < degree - tail; ++l) {
        if (prefixes > uint64_t(kMaxGridX)) return false;
        prefixes *= d;
    }
    const uint64_t wpp = (prefixes + kDeepLanes - 1) / kDeepLanes;
    return wpp <= uint64_t(kMaxGridX) / batch;
}

template <typename T, int D>
static hipError_t launch_fwd_d(const FwdParams& p, int degree)
{
    constexpr int TAIL = DeepTail<D>::value;
    const int M = degree - TAIL;
    if (M < 1 || degree > kDeepMaxDegree || p.nseg != 1) return hipErrorInvalidConfiguration;
    const int64_t P = ipow64(D, M);
    const int64_t wpp = (P + kDeepLanes - 1) / kDeepLanes;
    if (p.batch < 1 || wpp > kMaxGridX / p.batch) return hipErrorInvalidConfiguration;
    const size_t lds = (size_t(2) * M * kDeepLanes + kDeepMaxDegree + 1) * sizeof(T);
    hipError_t e = allow_lds(deep_fwd_kernel<T, D>, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((deep_fwd_kernel<T, D>), dim3(unsigned(p.batch * wpp)), dim3(kDeepLanes), lds, p.stream,
                       static_cast<const T*>(p.inc), static_cast<T*>(p.out), p.batch, p.L, degree, p.out_stride, p.scalar, P, wpp,
                       p.nonfinite);
    return hipGetLastError();
}

template <typename T, int D>
static hipError_t launch_bwd_d(const BwdParams& p, int degree)
{
    constexpr int TAIL = DeepTail<D>::value;
    const int M = degree - TAIL;
    if (M < 1 || degree > kDeepMaxDegree || p.nseg != 1) return hipErrorInvalidConfiguration;
    const int64_t P = ipow64(D, M);
    const int64_t wpp = (P + kDeepLanes - 1) / kDeepLanes;
    if (p.batch < 1 || wpp > kMaxGridX / p.batch) return hipErrorInvalidConfiguration;
    const size_t lds = (size_t(4) * M * kDeepLanes + kDeepMaxDegree + 1) * sizeof(T);
    hipError_t e = allow_lds(deep_bwd_kernel<T, D>, lds);
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL((deep_bwd_kernel<T, D>), dim3(unsigned(p.batch * wpp)), dim3(kDeepLanes), lds, p.stream,
                       static_cast<const T*>(p.inc), static_cast<const T*>(p.sig), static_cast<const T*>(p.gsig),
                       static_cast<T*>(p.dzinc), p.batch, p.L, degree, p.sig_stride, p.scalar, P, wpp);
    return hipGetLastError();
}

template <typename T>
hipError_t launch_deep_fwd(const FwdParams& p, int degree)
{
    switch (p.d) {
        case 2: return launch_fwd_d<T, 2>(p, degree);
        case 3: return launch_fwd_d<T, 3>(p, degree);
        case 4: return launch_fwd_d<T, 4>(p, degree);
        default: return hipErrorInvalidConfiguration;
    }
}

template <typename T>
hipError_t launch_deep_bwd(const BwdParams& p, int degree)
{
    switch (p.d) {
        case 2: return launch_bwd_d<T, 2>(p, degree);
        case 3: return launch_bwd_d<T, 3>(p, degree);
        case 4: return launch_bwd_d<T, 4>(p, degree);
        default: return hipErrorInvalidConfiguration;
    }
}

template hipError_t launch_deep_fwd<float>(const FwdParams&, int);
template hipError_t launch_deep_fwd<double>(const FwdParams&, int);
template hipError_t launch_deep_bwd<float>(const BwdParams&, int);
template hipError_t launch_deep_bwd<double>(const BwdParams&, int);

}  // namespace sigamd
