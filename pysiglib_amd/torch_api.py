"""Autograd wrapper (pysiglib/torch_api/torch_api.py:76-117): forward saves (path, signature),
backward un-multiplies the saved signature instead of storing per-step states."""
import torch

from .sig import sig as _sig_forward
from .sig import sig_backprop as _sig_backprop


class Sig(torch.autograd.Function):
    @staticmethod
    def forward(ctx, path, degree, time_aug, lead_lag, end_time, horner, scalar_term, n_jobs):
        out = _sig_forward(path, degree, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time, horner=horner,
                           scalar_term=scalar_term, n_jobs=n_jobs)
        ctx.save_for_backward(path, out)
        ctx.args = (degree, time_aug, lead_lag, end_time, n_jobs)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        path, out = ctx.saved_tensors
        degree, time_aug, lead_lag, end_time, n_jobs = ctx.args
        grad = _sig_backprop(path, out, grad_output, degree, time_aug=time_aug, lead_lag=lead_lag,
                             end_time=end_time, n_jobs=n_jobs)
        return grad, None, None, None, None, None, None, None


def sig(path, degree, *, time_aug=False, lead_lag=False, end_time=1., horner=True, scalar_term=False, n_jobs=1):
    """Differentiable ``sig``."""
    return Sig.apply(path, degree, time_aug, lead_lag, end_time, horner, scalar_term, n_jobs)


signature = sig


class SigCombine(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sig1, sig2, dimension, degree, time_aug, lead_lag):
        from .ops import sig_combine as _combine
        out = _combine(sig1, sig2, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
        ctx.save_for_backward(sig1, sig2)
        ctx.args = (dimension, degree, time_aug, lead_lag)
        return out

    @staticmethod
    def backward(ctx, grad_output):
        from .ops import sig_combine_backprop as _combine_backprop
        sig1, sig2 = ctx.saved_tensors
        dimension, degree, time_aug, lead_lag = ctx.args
        d1, d2 = _combine_backprop(grad_output, sig1, sig2, dimension, degree, time_aug=time_aug, lead_lag=lead_lag)
        return d1, d2, None, None, None, None


def sig_combine(sig1, sig2, dimension, degree, *, time_aug=False, lead_lag=False, n_jobs=1):
    """Differentiable ``sig_combine``."""
    return SigCombine.apply(sig1, sig2, dimension, degree, time_aug, lead_lag)


class TransformPath(torch.autograd.Function):
    @staticmethod
    def forward(ctx, path, time_aug, lead_lag, end_time):
        from .ops import transform_path as _transform
        ctx.args = (time_aug, lead_lag, end_time)
        return _transform(path, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time)

    @staticmethod
    def backward(ctx, grad_output):
        from .ops import transform_path_backprop as _transform_backprop
        time_aug, lead_lag, end_time = ctx.args
        return _transform_backprop(grad_output, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time), None, None, None


def transform_path(path, *, time_aug=False, lead_lag=False, end_time=1., n_jobs=1):
    """Differentiable ``transform_path``."""
    if (not time_aug) and (not lead_lag):
        return path
    return TransformPath.apply(path, time_aug, lead_lag, end_time)


class SigJoin(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sig, displacement, dimension, degree, prepend):
        from .ops import sig_join as _join
        ctx.save_for_backward(sig, displacement)
        ctx.args = (dimension, degree, prepend)
        return _join(sig, displacement, dimension, degree, prepend=prepend)

    @staticmethod
    def backward(ctx, grad_output):
        from .ops import sig_join_backprop as _join_backprop
        sig, displacement = ctx.saved_tensors
        dimension, degree, prepend = ctx.args
        d_sig, d_disp = _join_backprop(grad_output, sig, displacement, dimension, degree, prepend=prepend)
        return d_sig, d_disp, None, None, None


def sig_join(sig, displacement, dimension, degree, *, prepend=False, n_jobs=1):
    """Differentiable ``sig_join``."""
    return SigJoin.apply(sig, displacement, dimension, degree, bool(prepend))


class SigCoef(torch.autograd.Function):
    @staticmethod
    def forward(ctx, path, words, time_aug, lead_lag, end_time):
        from .coef import sig_coef as _coef
        coefs = _coef(path, words, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time, prefixes=True)
        ctx.save_for_backward(coefs, path)
        ctx.args = (words, time_aug, lead_lag, end_time)
        return coefs

    @staticmethod
    def backward(ctx, grad_output):
        from .coef import sig_coef_backprop as _coef_backprop
        coefs, path = ctx.saved_tensors
        words, time_aug, lead_lag, end_time = ctx.args
        grad = _coef_backprop(path, words, coefs, grad_output, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time)
        return grad, None, None, None, None


def sig_coef(path, words, *, time_aug=False, lead_lag=False, end_time=1., prefixes=False, n_jobs=1):
    """Differentiable ``sig_coef``: computes the prefixes layout and, without ``prefixes``, keeps each word's last
    entry (pysiglib/torch_api/torch_api.py:156-202)."""
    coefs = SigCoef.apply(path, words, time_aug, lead_lag, end_time)
    if prefixes:
        return coefs
    word_list = [words] if isinstance(words, tuple) else words
    ends, pos = [], 0
    for w in word_list:
        pos += max(len(w), 1)
        ends.append(pos - 1)
    return coefs[..., ends].contiguous()


class SigToLogSig(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sig_, dimension, degree, time_aug, lead_lag, method):
        from .log_sig import sig_to_log_sig as _to_log
        ctx.save_for_backward(sig_)
        ctx.args = (dimension, degree, time_aug, lead_lag, method)
        return _to_log(sig_, dimension, degree, time_aug=time_aug, lead_lag=lead_lag, method=method)

    @staticmethod
    def backward(ctx, grad_output):
        from .log_sig import sig_to_log_sig_backprop as _to_log_backprop
        (sig_,) = ctx.saved_tensors
        dimension, degree, time_aug, lead_lag, method = ctx.args
        grad = _to_log_backprop(sig_, grad_output, dimension, degree, time_aug=time_aug, lead_lag=lead_lag, method=method)
        return grad, None, None, None, None, None


def sig_to_log_sig(sig_, dimension, degree, *, time_aug=False, lead_lag=False, method=1, n_jobs=1):
    """Differentiable ``sig_to_log_sig``."""
    return SigToLogSig.apply(sig_, dimension, degree, time_aug, lead_lag, method)


def log_sig(path, degree, *, time_aug=False, lead_lag=False, end_time=1., method=1, scalar_term=False, n_jobs=1):
    """Differentiable ``log_sig``: the differentiable signature followed by the differentiable ``sig_to_log_sig``."""
    sig_ = sig(path, degree, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time, scalar_term=scalar_term)
    return sig_to_log_sig(sig_, path.shape[-1], degree, time_aug=time_aug, lead_lag=lead_lag, method=method)
