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
