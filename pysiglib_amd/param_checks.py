"""Argument checks with the reference's behaviour (pysiglib/param_checks.py:32-104)."""
import warnings

import numpy as np
import torch

SUPPORTED = (np.float32, np.float64, torch.float32, torch.float64)


def _type_name(t):
    return getattr(t, "__name__", str(t))


def check_type(value, name, expected):
    if not isinstance(value, expected):
        raise TypeError(name + " must be of type " + _type_name(expected) + ", got " + _type_name(type(value)) + " instead")


def check_array(value, name):
    if not isinstance(value, (np.ndarray, torch.Tensor)):
        raise TypeError(name + " must be of type ndarray or Tensor, got " + _type_name(type(value)) + " instead")


def check_non_neg(value, name):
    if value < 0:
        raise ValueError(name + " must be a non-negative integer, got " + name + " = " + str(value))


def check_n_jobs(n_jobs):
    check_type(n_jobs, "n_jobs", int)
    if n_jobs == 0:
        raise ValueError("n_jobs cannot be 0")


def check_dtype(arr, name):
    if arr.dtype not in SUPPORTED:
        raise TypeError(name + ".dtype must be float32 or float64, got " + str(arr.dtype) + " instead")


_warned = False
_MESSAGE = ("Detected a non-contiguous or view-based array. Such arrays will be cloned to ensure safe access. "
            "To avoid this overhead, pass arrays that are both contiguous and own their data. "
            "This warning will only appear once per session.")


def own_contiguous(arr):
    """Views, non-contiguous and stride-0 arrays are cloned (one warning per session)."""
    global _warned
    if isinstance(arr, torch.Tensor):
        needs = arr._base is not None or not arr.is_contiguous() or any(s == 0 for s in arr.stride())
        if needs:
            if not _warned:
                warnings.warn(_MESSAGE, stacklevel=4)
                _warned = True
            return arr.clone().contiguous()
        return arr
    if isinstance(arr, np.ndarray):
        if arr.base is not None or not arr.flags["C_CONTIGUOUS"]:
            if not _warned:
                warnings.warn(_MESSAGE, stacklevel=4)
                _warned = True
            return np.ascontiguousarray(arr.copy())
        return arr
    raise TypeError("expected a numpy.ndarray or torch.Tensor")


def check_word(word, max_val, word_name):
    """A word is a tuple of integer letters in [0, max_val) (pysiglib/param_checks.py:124-133)."""
    if not isinstance(word, tuple):
        raise TypeError(word_name + " must be a tuple of integers.")
    for i in word:
        if not isinstance(i, int):
            raise TypeError(word_name + " must be a tuple of integers. Found element of type " + str(type(i)) + " instead.")
        if not 0 <= i < max_val:
            raise ValueError(word_name + " must only contain letters in the range [0, " + str(max_val) + ")")


def check_word_or_word_list(param, max_val, param_name):
    """Returns the words as a list (pysiglib/param_checks.py:135-153)."""
    try:
        if isinstance(param, tuple):
            check_word(param, max_val, param_name)
            return [param]
        if isinstance(param, list):
            for word in param:
                check_word(word, max_val, "Every word in " + param_name)
            return param
    except Exception as e:
        raise type(e)("Error processing words: " + str(e)) from e
    raise TypeError(param_name + " must be a tuple of integers or a list of tuples of integers.")
