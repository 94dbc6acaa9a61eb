"""Log signatures: ``sig_to_log_sig``, ``sig_to_log_sig_backprop``, ``log_sig``, ``prepare_log_sig``, ``clear_cache`` with the
reference's signatures (pysiglib/log_sig.py:93-470, pysiglib/log_sig_backprop.py:30-137) for GPU tensors.  Method 0 is the
expanded tensor logarithm; methods 1 and 2 are its coordinates at the Lyndon words resp. in the Lyndon basis and need
``prepare_log_sig`` first, as in the reference.  Method 3 (BCH, straight from the path) is not part of this build."""
import torch

from ._loader import CUSIG, CUSIG_SIG_TO_LOG_SIG, CUSIG_SIG_TO_LOG_SIG_BACKPROP
from .data_handlers import SigInput, empty_like_input, on_device
from .error_codes import err_msg
from .ops import _same
from .param_checks import check_n_jobs, check_non_neg, check_type
from .sig import sig
from .sig_length import aug_dim, infer_scalar_term, log_sig_length, sig_length


def _check_method(method, who, allow_bch=False):
    check_type(method, "method", int)
    if method < 0 or method > 3:
        raise ValueError("method must be one of 0, 1, 2 or 3. Got " + str(method) + " instead.")
    if method == 3:
        if not allow_bch:
            raise ValueError("method=3 is not supported in " + who + ". Use log_sig(path, degree, method=3) instead.")
        raise NotImplementedError(who + ": method=3 (BCH) is not implemented in this build; use method 0, 1 or 2")


def prepare_log_sig(dimension, degree, method, *, time_aug=False, lead_lag=False, use_disk=False, device="cuda"):
    """Prepares the Lyndon tables of methods 1 and 2 on the current GPU (method 2 also serves method 1; method 0
    needs nothing).  ``use_disk`` is accepted for interface compatibility: tables are rebuilt in memory."""
    check_type(dimension, "dimension", int)
    check_type(degree, "degree", int)
    _check_method(method, "prepare_log_sig", allow_bch=True)
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(device, "device", str)
    if device not in ("cpu", "cuda", "both"):
        raise ValueError("device must be 'cpu', 'cuda', or 'both'")
    if method == 0 or device == "cpu":
        return
    code = CUSIG.prepare_log_sig_cuda(aug_dim(dimension, time_aug, lead_lag), degree, method, bool(use_disk))
    if code:
        raise Exception("Error in pysiglib.prepare_log_sig: " + err_msg(code))


def clear_cache(*, use_disk=False, device="both"):
    """Drops every prepared table."""
    check_type(device, "device", str)
    if device not in ("cpu", "cuda", "both"):
        raise ValueError("device must be 'cpu', 'cuda', or 'both'")
    if device == "cpu":
        return
    code = CUSIG.clear_cache_cuda(bool(use_disk))
    if code:
        raise Exception("Error in pysiglib.clear_cache: " + err_msg(code))


def _checks(dimension, degree, time_aug, lead_lag):
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)


def sig_to_log_sig(sig_, dimension, degree, *, time_aug=False, lead_lag=False, method=1, n_jobs=1):
    """Log signature from a signature.  method 0: the layout of the input (scalar slot, if any, 0); methods 1, 2:
    ``log_sig_length`` coordinates."""
    _checks(dimension, degree, time_aug, lead_lag)
    _check_method(method, "sig_to_log_sig")
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig_, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    data = SigInput(sig_, n, "sig")
    out, out_ptr = empty_like_input(data, (log_sig_length(d, degree) if method else n,))
    if data.batch_size == 0:
        return out
    check_n_jobs(n_jobs)
    with on_device(data.device):
        code = CUSIG_SIG_TO_LOG_SIG[data.dtype](data.data_ptr, out_ptr, data.batch_size, d, degree, method, scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_to_log_sig: " + err_msg(code))
    return out


def sig_to_log_sig_backprop(sig_, log_sig_derivs, dimension, degree, *, time_aug=False, lead_lag=False, method=1, n_jobs=1):
    """Gradient w.r.t. the signature given the gradient w.r.t. ``sig_to_log_sig(sig, ..., method=method)``."""
    _checks(dimension, degree, time_aug, lead_lag)
    _check_method(method, "sig_to_log_sig_backprop")
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig_, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    data = SigInput(sig_, n, "sig")
    derivs = SigInput(log_sig_derivs, log_sig_length(d, degree) if method else n, "log_sig_derivs")
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
    _check_method(method, "log_sig", allow_bch=True)
    sig_ = sig(path, degree, scalar_term=scalar_term, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time, horner=True,
               correction=correction, n_jobs=n_jobs)
    return sig_to_log_sig(sig_, path.shape[-1], degree, time_aug=time_aug, lead_lag=lead_lag, method=method, n_jobs=n_jobs)
