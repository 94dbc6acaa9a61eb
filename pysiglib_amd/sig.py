"""``sig`` / ``sig_backprop`` with the reference's signatures and error behaviour
(pysiglib/sig.py:128-312, pysiglib/sig_backprop.py:128-256), driving the HIP library."""
import warnings

import torch

from ._loader import CUSIG, CUSIG_SIG_BACKPROP, CUSIG_SIGNATURE
from .data_handlers import PathInput, SigInput, empty_like_input, on_device
from .error_codes import err_msg
from .param_checks import check_n_jobs, check_non_neg, check_type
from .sig_length import infer_scalar_term, sig_length


def _no_correction(correction):
    if correction is None:
        return
    n = correction.size if hasattr(correction, "size") and not callable(correction.size) else correction.numel()
    if n != 0:
        raise NotImplementedError("per-segment correction is not implemented in pysiglib_amd")


def sig(path, degree, *, time_aug=False, lead_lag=False, end_time=1., horner=True, scalar_term=False,
        correction=None, n_jobs=1):
    """Truncated signature of a path ``(length, dimension)`` or batch ``(..., length, dimension)``.

    Returns a tensor ``(..., S)`` on the input's device; ``S`` excludes the leading 1 unless
    ``scalar_term=True``.  ``n_jobs`` is accepted for interface compatibility (the GPU ignores it).
    """
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(horner, "horner", bool)
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    check_n_jobs(n_jobs)
    data = PathInput(path, time_aug, lead_lag, end_time, "path")
    _no_correction(correction)
    n = sig_length(data.dimension, degree, scalar_term=scalar_term)
    out, out_ptr = empty_like_input(data, (n,))
    if data.batch_size == 0:
        return out
    with on_device(data.device):
        code = CUSIG_SIGNATURE[data.dtype](
            data.data_ptr, out_ptr, data.batch_size, data.data_dimension, data.data_length, degree,
            time_aug, lead_lag, end_time, horner, scalar_term, None, 0, 0, 0)
    if code:
        raise Exception("Error in pysiglib.sig: " + err_msg(code))
    # the kernels that store the signature report NaN / Inf themselves; scan only when they could not
    reported = CUSIG.cusig_amd_last_sig_nonfinite()
    if reported == 1 or (reported < 0 and not torch.isfinite(out).all().item()):
        warnings.warn(
            "sig produced NaN or Inf values. This is typically caused by paths with large increments, "
            "leading to numerical overflow. Consider normalizing your paths.", RuntimeWarning, stacklevel=2)
    return out


signature = sig


def sig_backprop(path, sig, sig_derivs, degree, *, time_aug=False, lead_lag=False, end_time=1.,
                 correction=None, n_jobs=1):
    """Gradient w.r.t. ``path`` given ``sig = sig(path, degree, ...)`` and the loss gradient ``sig_derivs``
    (same shape as ``sig``; whether the scalar term is present is inferred from the width of ``sig``)."""
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    pdata = PathInput(path, time_aug, lead_lag, end_time, "path")
    _no_correction(correction)
    scalar_term = infer_scalar_term(sig, pdata.data_dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(pdata.dimension, degree, scalar_term=scalar_term)
    sdata = SigInput(sig, n, "sig")
    gdata = SigInput(sig_derivs, n, "sig_derivs")
    if sdata.dtype != gdata.dtype:
        raise ValueError("sig, sig_derivs must have the same dtype")
    if sdata.batch_shape != gdata.batch_shape:
        raise ValueError("sig, sig_derivs have different batch shapes")
    if sdata.device != gdata.device:
        raise ValueError("sig, sig_derivs must be on the same device")
    if pdata.dtype != sdata.dtype:
        raise ValueError("path, sig and sig_derivs must have the same dtype")
    out, out_ptr = empty_like_input(pdata, (pdata.data_length, pdata.data_dimension))
    if pdata.batch_size == 0:
        return out
    if pdata.batch_shape != sdata.batch_shape:
        raise ValueError("path, sig and sig_derivs must have the same batch shape")
    if pdata.device != sdata.device:
        raise ValueError("path, sig and sig_derivs must be on the same device")
    check_n_jobs(n_jobs)
    with on_device(pdata.device):
        code = CUSIG_SIG_BACKPROP[pdata.dtype](
            pdata.data_ptr, out_ptr, gdata.data_ptr, sdata.data_ptr, pdata.batch_size, pdata.data_dimension,
            pdata.data_length, degree, time_aug, lead_lag, end_time, scalar_term, None, 0, 0, 0)
    if code:
        raise Exception("Error in pysiglib.sig_backprop: " + err_msg(code))
    return out
