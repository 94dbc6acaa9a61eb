// Adjoint of the Chen product, shared by sig_combine_backprop, sig_join_backprop and the tensor logarithm's backward
// pass, plus the row layout helper of the signature-shaped operators.
#pragma once
#include <hip/hip_runtime.h>

#include <stdexcept>
#include <string>

#include "sig_host.h"

namespace sigamd {

constexpr int kCombMaxLevels = 64;      // highest degree the adjoint of the Chen product takes

struct SigShape {
    uint64_t n_coef, stride;
    int off;
};

static SigShape sig_shape(uint64_t dimension, uint64_t degree, bool scalar_term, const char* who)
{
    if (dimension == 0) throw std::invalid_argument(std::string(who) + " received dimension 0");
    if (dimension > 0x3fffffff || degree > 0x7fffffff) throw std::invalid_argument(std::string(who) + ": shape out of range");
    const uint64_t full = sig_length_u64(dimension, degree);
    if (full == 0) throw std::overflow_error("signature length overflows 64 bits");
    SigShape s;
    s.n_coef = full - 1;
    s.stride = scalar_term ? full : full - 1;
    s.off = scalar_term ? 1 : 0;
    return s;
}

// how the rows of dC are found when they differ from the other operands' layout
struct SharedRows {
    int64_t share = 1;      // consecutive items reading one row
    int64_t stride = -1;    // < 0: same stride and offset as the other operands
    int off = 0;
};

// B = exp(z) and the caller wants dz (zeroed beforehand) rather than dB: the right factor's kernel may add the terms
// of the levels above `level` straight into dz.  On return dB holds, at `level`, the row on which the adjoint of exp
// truncated at `level` gives the remaining terms (levels above it are not written); level = degree: nothing folded.
template <typename T>
struct ExpFold {
    const T* z = nullptr;   // (batch, dimension)
    T* dz = nullptr;
    int level = 0;
};

// launches the adjoint of the Chen product on `stream` (defined in sig_chen_adjoint.hip for float and double).
// identity: bit 0 keeps the dC_k[u] term of dA, bit 1 the dC_t[w] term of dB; a gradient without that term is zero at
// the top level, which the streaming kernels then leave unwritten.  families = 1 computes dA only (dB and A are not
// touched)
template <typename T>
void launch_combine_bwd(const T* dC, T* dA, T* dB, const T* A, const T* B, uint64_t batch, uint64_t dimension,
                        uint64_t degree, const SigShape& s, hipStream_t stream, int identity = 3,
                        SharedRows dc = SharedRows(), int families = 2, ExpFold<T>* fold = nullptr);
extern template void launch_combine_bwd<float>(const float*, float*, float*, const float*, const float*, uint64_t, uint64_t,
                                               uint64_t, const SigShape&, hipStream_t, int, SharedRows, int, ExpFold<float>*);
extern template void launch_combine_bwd<double>(const double*, double*, double*, const double*, const double*, uint64_t,
                                                uint64_t, uint64_t, const SigShape&, hipStream_t, int, SharedRows, int,
                                                ExpFold<double>*);

}  // namespace sigamd
