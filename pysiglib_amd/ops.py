"""Operators either side of the signature: ``sig_combine``, ``sig_join``, ``linear_sig``, ``transform_path`` and their
backward passes, with the reference's signatures (pysiglib/sig.py:28-126, pysiglib/sig_join.py,
pysiglib/sig_join_backprop.py, pysiglib/linear_sig.py, pysiglib/transform_path.py:28-103,
pysiglib/transform_path_backprop.py, pysiglib/torch_api/torch_api.py) for GPU tensors."""
import torch

from ._loader import (CUSIG_LINEAR_SIG, CUSIG_SIG_COMBINE, CUSIG_SIG_COMBINE_BACKPROP, CUSIG_SIG_JOIN,
                      CUSIG_SIG_JOIN_BACKPROP, CUSIG_TRANSFORM_PATH, CUSIG_TRANSFORM_PATH_BACKPROP)
from .data_handlers import PathInput, SigInput, empty_like_input, on_device
from .error_codes import err_msg
from .param_checks import check_n_jobs, check_non_neg, check_type
from .sig_length import aug_dim, infer_scalar_term, sig_length


def _same(inputs, names):
    first = inputs[0]
    for other in inputs[1:]:
        if other.dtype != first.dtype:
            raise ValueError(", ".join(names) + " must have the same dtype")
        if other.batch_shape != first.batch_shape:
            raise ValueError(", ".join(names) + " have different batch shapes")
        if other.device != first.device:
            raise ValueError(", ".join(names) + " must be on the same device")


def sig_combine(sig1, sig2, dimension, degree, *, time_aug=False, lead_lag=False, n_jobs=1):
    """Chen product: the signature of the concatenation of two paths from their signatures."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_n_jobs(n_jobs)
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig1, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    a, b = SigInput(sig1, n, "sig1"), SigInput(sig2, n, "sig2")
    _same([a, b], ["sig1", "sig2"])
    out, out_ptr = empty_like_input(a, (n,))
    if a.batch_size == 0:
        return out
    with on_device(a.device):
        code = CUSIG_SIG_COMBINE[a.dtype](a.data_ptr, b.data_ptr, out_ptr, a.batch_size, d, degree, scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_combine: " + err_msg(code))
    return out


def sig_combine_backprop(derivs, sig1, sig2, dimension, degree, *, time_aug=False, lead_lag=False, n_jobs=1):
    """Gradients w.r.t. ``sig1`` and ``sig2`` given the gradient w.r.t. ``sig_combine(sig1, sig2)``."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_n_jobs(n_jobs)
    d = aug_dim(dimension, time_aug, lead_lag)
    scalar_term = infer_scalar_term(sig1, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
    n = sig_length(d, degree, scalar_term=scalar_term)
    g, a, b = SigInput(derivs, n, "derivs"), SigInput(sig1, n, "sig1"), SigInput(sig2, n, "sig2")
    _same([g, a, b], ["derivs", "sig1", "sig2"])
    d1, d1_ptr = empty_like_input(a, (n,))
    d2, d2_ptr = empty_like_input(a, (n,))
    if a.batch_size == 0:
        return d1, d2
    with on_device(a.device):
        code = CUSIG_SIG_COMBINE_BACKPROP[a.dtype](g.data_ptr, d1_ptr, d2_ptr, a.data_ptr, b.data_ptr, a.batch_size, d,
                                                   degree, scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_combine_backprop: " + err_msg(code))
    return d1, d2


def transform_path(path, *, time_aug=False, lead_lag=False, end_time=1., n_jobs=1):
    """Applies the lead-lag transformation and/or appends time as the last channel."""
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    if (not time_aug) and (not lead_lag):
        return path
    check_n_jobs(n_jobs)
    data = PathInput(path, time_aug, lead_lag, end_time, "path")
    if time_aug and data.data_length < 2:
        raise ValueError(f"transform_path(time_aug=True) requires path length >= 2, got {data.data_length}. ")
    out, out_ptr = empty_like_input(data, (data.length, data.dimension))
    if data.batch_size == 0:
        return out
    with on_device(data.device):
        code = CUSIG_TRANSFORM_PATH[data.dtype](data.data_ptr, out_ptr, data.batch_size, data.data_dimension,
                                                data.data_length, time_aug, lead_lag, end_time)
    if code:
        raise Exception("Error in pysiglib.transform_path: " + err_msg(code))
    return out


def transform_path_backprop(derivs, *, time_aug=False, lead_lag=False, end_time=1., n_jobs=1):
    """Gradient w.r.t. the raw path given the gradient w.r.t. ``transform_path(path, ...)``."""
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    if (not time_aug) and (not lead_lag):
        return derivs
    check_n_jobs(n_jobs)
    data = PathInput(derivs, False, False, end_time, "derivs")
    t_len, t_dim = data.data_length, data.data_dimension
    dim = t_dim - (1 if time_aug else 0)
    if lead_lag:
        if dim % 2 or t_len % 2 == 0:
            raise ValueError("derivs does not have the shape of a lead-lag transformed path")
        dim //= 2
        length = (t_len + 1) // 2
    else:
        length = t_len
    if dim < 1:
        raise ValueError("derivs does not have the shape of a transformed path")
    out, out_ptr = empty_like_input(data, (length, dim))
    if data.batch_size == 0:
        return out
    with on_device(data.device):
        code = CUSIG_TRANSFORM_PATH_BACKPROP[data.dtype](data.data_ptr, out_ptr, data.batch_size, dim, length, time_aug,
                                                         lead_lag, end_time)
    if code:
        raise Exception("Error in pysiglib.transform_path_backprop: " + err_msg(code))
    return out


def linear_sig(displacement, dimension, degree, *, scalar_term=False, n_jobs=1):
    """Signature of the straight line with the given displacement(s), shape (..., dimension)."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_type(scalar_term, "scalar_term", bool)
    check_n_jobs(n_jobs)
    n = sig_length(dimension, degree, scalar_term=scalar_term)
    z = SigInput(displacement, dimension, "displacement")
    out, out_ptr = empty_like_input(z, (n,))
    if z.batch_size == 0:
        return out
    with on_device(z.device):
        code = CUSIG_LINEAR_SIG[z.dtype](z.data_ptr, out_ptr, z.batch_size, dimension, degree, scalar_term)
    if code:
        raise Exception("Error in pysiglib.linear_sig: " + err_msg(code))
    return out


def sig_join(sig, displacement, dimension, degree, *, prepend=False, n_jobs=1):
    """Extends each signature by one straight-line segment: S(x * v), or S(v * x) with ``prepend=True``."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_n_jobs(n_jobs)
    scalar_term = infer_scalar_term(sig, dimension, degree)
    n = sig_length(dimension, degree, scalar_term=scalar_term)
    a, z = SigInput(sig, n, "sig"), SigInput(displacement, dimension, "displacement")
    _same([a, z], ["sig", "displacement"])
    out, out_ptr = empty_like_input(a, (n,))
    if a.batch_size == 0:
        return out
    with on_device(a.device):
        code = CUSIG_SIG_JOIN[a.dtype](a.data_ptr, z.data_ptr, out_ptr, a.batch_size, dimension, degree, bool(prepend),
                                       scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_join: " + err_msg(code))
    return out


def sig_join_backprop(d_out, sig, displacement, dimension, degree, *, prepend=False, n_jobs=1):
    """Gradients w.r.t. ``sig`` and ``displacement`` given the gradient w.r.t. ``sig_join(sig, displacement)``."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(degree, "degree", int)
    check_non_neg(degree, "degree")
    check_n_jobs(n_jobs)
    scalar_term = infer_scalar_term(sig, dimension, degree)
    n = sig_length(dimension, degree, scalar_term=scalar_term)
    g, a, z = SigInput(d_out, n, "d_out"), SigInput(sig, n, "sig"), SigInput(displacement, dimension, "displacement")
    _same([g, a, z], ["d_out", "sig", "displacement"])
    d_sig, d_sig_ptr = empty_like_input(g, (n,))
    d_disp, d_disp_ptr = empty_like_input(g, (dimension,))
    if g.batch_size == 0:
        return d_sig, d_disp
    with on_device(g.device):
        code = CUSIG_SIG_JOIN_BACKPROP[g.dtype](g.data_ptr, d_sig_ptr, d_disp_ptr, a.data_ptr, z.data_ptr, g.batch_size,
                                                dimension, degree, bool(prepend), scalar_term)
    if code:
        raise Exception("Error in pysiglib.sig_join_backprop: " + err_msg(code))
    return d_sig, d_disp
