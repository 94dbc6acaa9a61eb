"""Coefficients of selected words: ``sig_coef``, ``sig_coef_backprop``, ``extract_sig_coef`` with the reference's
signatures (pysiglib/sig_coef.py, pysiglib/sig_coef_backprop.py, pysiglib/words.py:135-154) for GPU tensors."""
from ctypes import POINTER, c_uint64, cast

import torch

from ._loader import CUSIG_SIG_COEF, CUSIG_SIG_COEF_BACKPROP
from .data_handlers import PathInput, SigInput, empty_like_input, on_device
from .error_codes import err_msg
from .ops import _same, transform_path, transform_path_backprop
from .param_checks import check_n_jobs, check_non_neg, check_type, check_word, check_word_or_word_list
from .sig_length import aug_dim


def word_to_idx(word, dimension, degree, *, scalar_term=False):
    """Index of ``word`` in a flattened signature of the given truncation degree."""
    check_type(dimension, "dimension", int)
    check_type(degree, "degree", int)
    check_type(scalar_term, "scalar_term", bool)
    check_word(word, dimension, "word")
    if len(word) > degree:
        raise ValueError("word exceeds the requested degree")
    if not word and not scalar_term:
        raise ValueError("The empty word has no index with scalar_term=False")
    idx = 0
    for letter in word:
        idx = idx * dimension + letter + 1
    return idx if scalar_term else idx - 1


def extract_sig_coef(sig, words, dimension, *, time_aug=False, lead_lag=False, scalar_term=False):
    """Picks the coefficients of ``words`` out of a signature or batch of signatures."""
    check_type(dimension, "dimension", int)
    check_non_neg(dimension, "dimension")
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    d = aug_dim(dimension, time_aug, lead_lag)
    words = check_word_or_word_list(words, d, "word")
    SigInput(sig, sig.shape[-1], "sig")
    degree = max((len(w) for w in words), default=0)
    return sig[..., [word_to_idx(w, d, degree, scalar_term=scalar_term) for w in words]]


def _device_words(words, device):
    flat = [i for w in words for i in w]
    letters = torch.tensor(flat if flat else [0], dtype=torch.int64, device=device)      # same bits as uint64
    degrees = torch.tensor([len(w) for w in words], dtype=torch.int64, device=device)
    return letters, degrees


def _u64(t):
    return cast(t.data_ptr(), POINTER(c_uint64))


def sig_coef(path, words, *, time_aug=False, lead_lag=False, end_time=1., prefixes=False, n_jobs=1):
    """Signature coefficients of ``path`` at the given words, shape (..., num_words); with ``prefixes=True`` every word
    contributes the coefficients of all its non-empty prefixes."""
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    check_type(prefixes, "prefixes", bool)
    data = PathInput(path, time_aug, lead_lag, end_time, "path")
    if time_aug or lead_lag:
        transformed = transform_path(path, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time)
        return sig_coef(transformed, words, prefixes=prefixes, n_jobs=n_jobs)
    words = check_word_or_word_list(words, data.dimension, "word")
    if len(words) == 0:
        raise ValueError("words must be a non-empty list of multi-indices.")
    row = sum((len(w) if w else 1) for w in words) if prefixes else len(words)
    out, out_ptr = empty_like_input(data, (row,))
    if data.batch_size == 0:
        return out
    check_n_jobs(n_jobs)
    letters, degrees = _device_words(words, data.device)
    with on_device(data.device):
        code = CUSIG_SIG_COEF[data.dtype](data.data_ptr, out_ptr, _u64(letters), len(words), _u64(degrees), data.batch_size,
                                          data.data_dimension, data.data_length, prefixes)
    if code:
        raise Exception("Error in pysiglib.sig_coef: " + err_msg(code))
    return out


def sig_coef_backprop(path, words, coefs, derivs, *, time_aug=False, lead_lag=False, end_time=1., n_jobs=1):
    """Gradient w.r.t. ``path`` given the gradient w.r.t. ``sig_coef(path, words, prefixes=True)``; ``coefs`` is that
    forward result."""
    check_type(time_aug, "time_aug", bool)
    check_type(lead_lag, "lead_lag", bool)
    check_type(end_time, "end_time", float)
    data = PathInput(path, time_aug, lead_lag, end_time, "path")
    if time_aug or lead_lag:
        transformed = transform_path(path, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time)
        aug_grad = sig_coef_backprop(transformed, words, coefs, derivs, n_jobs=n_jobs)
        return transform_path_backprop(aug_grad, time_aug=time_aug, lead_lag=lead_lag, end_time=end_time)
    words = check_word_or_word_list(words, data.dimension, "word")
    row = sum((len(w) if w else 1) for w in words)
    if coefs.shape[-1] != row:
        raise ValueError("Expected coefs.shape[-1] == " + str(row) + ". Please make sure coefs was generated using prefixes=True.")
    c, g = SigInput(coefs, row, "coef"), SigInput(derivs, row, "deriv")
    _same([c, g], ["coef", "deriv"])
    if c.dtype != data.dtype or c.batch_shape != data.batch_shape or c.device != data.device:
        raise ValueError("path, coef and deriv must agree in dtype, batch shape and device")
    out, out_ptr = empty_like_input(data, (data.data_length, data.data_dimension))
    if data.batch_size == 0:
        return out
    check_n_jobs(n_jobs)
    letters, degrees = _device_words(words, data.device)
    with on_device(data.device):
        code = CUSIG_SIG_COEF_BACKPROP[data.dtype](data.data_ptr, out_ptr, c.data_ptr, g.data_ptr, _u64(letters), len(words),
                                                   _u64(degrees), data.batch_size, data.data_dimension, data.data_length)
    if code:
        raise Exception("Error in pysiglib.sig_coef_backprop: " + err_msg(code))
    return out
