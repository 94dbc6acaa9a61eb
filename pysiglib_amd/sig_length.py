"""Signature and log-signature sizes (pysiglib/sig_length.py:20-182)."""
from ._loader import CUSIG
from .param_checks import check_non_neg, check_type


def aug_dim(dimension, time_aug, lead_lag):
    return (2 * dimension if lead_lag else dimension) + (1 if time_aug else 0)


def sig_length(dimension, degree, *, time_aug=False, lead_lag=False, scalar_term=False):
    """Number of coefficients of a degree-``degree`` signature in ``dimension`` channels.

    With ``scalar_term=False`` (default) the leading 1 is not counted.
    Raises ValueError on 64-bit overflow.
    """
    check_type(dimension, "dimension", int)
    check_type(degree, "degree", int)
    check_non_neg(dimension, "dimension")
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    out = int(CUSIG.cusig_amd_sig_length(aug_dim(dimension, time_aug, lead_lag), degree))
    if out == 0:
        raise ValueError("Integer overflow encountered in sig_length")
    return out - (0 if scalar_term else 1)


def infer_scalar_term(sig, dimension, degree, time_aug=False, lead_lag=False):
    """True iff the last axis of ``sig`` includes the leading scalar 1."""
    full = sig_length(dimension, degree, time_aug=time_aug, lead_lag=lead_lag, scalar_term=True)
    actual = sig.shape[-1]
    if actual == full:
        return True
    if actual == full - 1:
        return False
    raise ValueError("sig has incompatible length " + str(actual) + " for dimension=" + str(dimension) +
                     ", degree=" + str(degree) + " (expected " + str(full) + " or " + str(full - 1) + ").")


def _mobius(n):
    result, p = 1, 2
    while p * p <= n:
        if n % p == 0:
            n //= p
            if n % p == 0:
                return 0
            result = -result
        p += 1
    return -result if n > 1 else result


def log_sig_length(dimension, degree, *, time_aug=False, lead_lag=False):
    """Number of Lyndon words of length at most ``degree`` over ``dimension`` letters: the length of a compressed
    (method 1, 2) log signature, ``sum_{i=1..N} 1/i sum_{x | i} mu(i / x) d^x`` (pysiglib/sig_length.py:97-163)."""
    check_type(dimension, "dimension", int)
    check_type(degree, "degree", int)
    check_non_neg(dimension, "dimension")
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    d = aug_dim(dimension, time_aug, lead_lag)
    total = 0
    for i in range(1, degree + 1):
        total += sum(_mobius(i // x) * d ** x for x in range(1, i + 1) if i % x == 0) // i
    return total
