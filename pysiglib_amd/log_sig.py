"""Log signatures in expanded coordinates (method 0): ``sig_to_log_sig``, ``sig_to_log_sig_backprop``, ``log_sig`` with the
reference's signatures (pysiglib/log_sig.py:223-470, pysiglib/log_sig_backprop.py:30-137) for GPU tensors.  Methods 1-3
(Lyndon coordinates, BCH) rely on prepared tables this build does not carry and raise."""
import torch

from ._loader import CUSIG_SIG_TO_LOG_SIG, CUSIG_SIG_TO_LOG_SIG_BACKPROP
from .data_handlers import SigInput, empty_like_input, on_device
from .error_codes import err_msg
from .ops import _same
from .param_checks import check_n_jobs, check_non_neg, check_type
from .sig import sig
from .sig_length import aug_dim, infer_scalar_term, sig_length


def _check_method(method, who):
    check_type(method, "method", int)
    if method not in (0, 1, 2, 3):
        raise ValueError("method must be one of 0, 1, 2, 3")
    if method != 0:
        raise NotImplementedError(who + ": only method=0 (expanded tensor logarithm) is implemented in this build; "
                                  "methods 1-3 need the reference's prepared Lyndon / BCH tables")


def _checks(dimension, degree, time_aug, lead_lag):
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)


def sig_to_log_sig(sig_, dimension, degree, *, time_aug=False, lead_lag=False, method=1, n_jobs=1):
    """Log signature from a signature; the result has the layout of the input (scalar slot, if any, 0)."""
    _checks(dimension, degree, time_aug, lead_lag)
    _check_method(method, "sig_to_log_sig")
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig_, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    data = SigInput(sig_, n, "sig")
    out, out_ptr = empty_like_input(data, (n,))
    if data.batch_size == 0:
        return out
    check_n_jobs(n_jobs)
    with on_device(data.device):
        code = CUSIG_SIG_TO_LOG_SIG[data.dtype](data.data_ptr, out_ptr, data.batch_size, d, degree, method, scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_to_log_sig: " + err_msg(code))
    return out


def sig_to_log_sig_backprop(sig_, log_sig_derivs, dimension, degree, *, time_aug=False, lead_lag=False, method=1, n_jobs=1):
    """Gradient w.r.t. the signature given the gradient w.r.t. ``sig_to_log_sig(sig)``."""
    _checks(dimension, degree, time_aug, lead_lag)
    _check_method(method, "sig_to_log_sig_backprop")
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig_, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    data, derivs = SigInput(sig_, n, "sig"), SigInput(log_sig_derivs, n, "log_sig_derivs")
    if data.dtype != derivs.dtype:
        raise ValueError("sig and log_sig_derivs must have the same dtype")
    _same([data, derivs], ["sig", "log_sig_derivs"])
    out, out_ptr = empty_like_input(data, (n,))
    if data.batch_size == 0:
        return out
    check_n_jobs(n_jobs)
    with on_device(data.device):
        code = CUSIG_SIG_TO_LOG_SIG_BACKPROP[data.dtype](data.data_ptr, out_ptr, derivs.data_ptr, data.batch_size, d, degree,
                                                         method, scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_to_log_sig_backprop: " + err_msg(code))
    return out


def log_sig(path, degree, *, time_aug=False, lead_lag=False, end_time=1., method=1, scalar_term=False, correction=None,
            n_jobs=1):
    """Log signature of a path: the signature followed by ``sig_to_log_sig``."""
    _check_method(method, "log_sig")
    sig_ = sig(path, degree, scalar_term=scalar_term, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time, horner=True,
               correction=correction, n_jobs=n_jobs)
    return sig_to_log_sig(sig_, path.shape[-1], degree, time_aug=time_aug, lead_lag=lead_lag, method=method, n_jobs=n_jobs)
