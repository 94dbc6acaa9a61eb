"""Independent float64 torch statement of the mathematics, used to pin the oracle.

Nothing here follows the reference's (or the oracle's) loop structure: the
signature is the Chen product of segment exponentials built with explicit
outer products, and gradients come from torch autograd through that product.
"""
import itertools

import numpy as np
import torch


def augment(x, time_aug=False, lead_lag=False, end_time=1.0):
    """Differentiable lead-lag / time augmentation of a (B, len, d) tensor.

    lead-lag doubles the channels as [lag | lead] over 2*len-1 points where the
    lead channel moves first; time is appended last and runs linearly over the
    transformed length.
    """
    if lead_lag:
        rep = torch.repeat_interleave(x, 2, dim=1)          # x0 x0 x1 x1 ...
        lag = rep[:, :-1]                                    # x0 x0 x1 x1 ... x_{n-1}
        lead = rep[:, 1:]                                    # x0 x1 x1 x2 ... x_{n-1}
        x = torch.cat((lag, lead), dim=2)
    if time_aug:
        t = torch.linspace(0.0, end_time, x.shape[1], dtype=x.dtype, device=x.device)
        x = torch.cat((x, t.expand(x.shape[0], -1).unsqueeze(2)), dim=2)
    return x


def _segment_exp(z, degree):
    """levels 1..degree of exp(z) for z of shape (B, d): z^(x)k / k!"""
    levels = [z]
    for k in range(2, degree + 1):
        levels.append((levels[-1].unsqueeze(2) * z.unsqueeze(1)).reshape(z.shape[0], -1) / k)
    return levels


def _chen(a, b, degree):
    """levels of a (x) b where a, b are lists of level tensors (B, d^k), scalar terms 1"""
    out = []
    for t in range(1, degree + 1):
        acc = a[t - 1] + b[t - 1]
        for k in range(1, t):
            acc = acc + (a[k - 1].unsqueeze(2) * b[t - k - 1].unsqueeze(1)).reshape(a[0].shape[0], -1)
        out.append(acc)
    return out


def signature(x, degree):
    """(B, len, d) -> (B, d + d^2 + ... + d^degree), no scalar term."""
    inc = x[:, 1:] - x[:, :-1]
    sig = _segment_exp(inc[:, 0], degree)
    for s in range(1, inc.shape[1]):
        sig = _chen(sig, _segment_exp(inc[:, s], degree), degree)
    return torch.cat(sig, dim=1)


def signature_np(x, degree, **aug):
    single = x.ndim == 2
    t = torch.as_tensor(np.asarray(x, dtype=np.float64))
    if single:
        t = t[None]
    out = signature(augment(t, **aug), degree).numpy()
    return out[0] if single else out


def backprop_np(x, g, degree, **aug):
    """gradient of <g, signature(augment(x))> w.r.t. x, by autograd."""
    single = x.ndim == 2
    t = torch.tensor(np.asarray(x, dtype=np.float64), requires_grad=True)
    gt = torch.as_tensor(np.asarray(g, dtype=np.float64))
    tt, gg = (t[None], gt[None]) if single else (t, gt)
    s = signature(augment(tt, **aug), degree)
    (grad,) = torch.autograd.grad((s * gg).sum(), t)
    return grad.numpy()


def iterated_sums(x, degree):
    """Brute force for a piecewise-linear path, independent of Chen's identity:
    the level-k coefficient of word w is the sum over non-decreasing segment
    tuples s_1 <= ... <= s_k of prod dx[s_i][w_i] divided by the product of
    factorials of the run lengths of equal segment indices."""
    from math import factorial
    inc = np.diff(np.asarray(x, dtype=np.float64), axis=0)
    n, d = inc.shape
    out = []
    for k in range(1, degree + 1):
        lvl = np.zeros((d,) * k)
        for segs in itertools.combinations_with_replacement(range(n), k):
            w = 1.0
            run = 1
            for a, b in zip(segs, segs[1:]):
                if a == b:
                    run += 1
                else:
                    w /= factorial(run)
                    run = 1
            w /= factorial(run)
            term = np.array(w)
            for s in segs:
                term = np.multiply.outer(term, inc[s])
            lvl += term
        out.append(lvl.ravel())
    return np.concatenate(out)


def level_slices(d, degree, scalar_term=False):
    off = 1 if scalar_term else 0
    out = []
    for k in range(1, degree + 1):
        out.append(slice(off, off + d ** k))
        off += d ** k
    return out


def level_rel_err(got, ref, d, degree):
    """max over paths and levels of ||got_k - ref_k||_inf / ||ref_k||_inf"""
    got = np.asarray(got, dtype=np.float64).reshape(-1, got.shape[-1])
    ref = np.asarray(ref, dtype=np.float64).reshape(-1, ref.shape[-1])
    worst = 0.0
    for sl in level_slices(d, degree):
        num = np.abs(got[:, sl] - ref[:, sl]).max(axis=1)
        den = np.maximum(np.abs(ref[:, sl]).max(axis=1), np.finfo(np.float64).tiny)
        worst = max(worst, float((num / den).max()))
    return worst
