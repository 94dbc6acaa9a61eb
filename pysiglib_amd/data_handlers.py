"""Marshalling of path / signature arguments (pysiglib/data_handlers.py:50-189).

This package drives the GPU library only: NumPy inputs and CPU tensors are
rejected with a clear error instead of being routed to a CPU implementation.
"""
from ctypes import POINTER, cast
from math import prod

import numpy as np
import torch

from ._loader import DTYPES
from .param_checks import check_array, check_dtype, own_contiguous


def _require_gpu(arr, name):
    if isinstance(arr, np.ndarray) or arr.device.type != "cuda":
        raise RuntimeError(
            name + " must be a torch tensor on the GPU: pysiglib_amd ships the MI355X path only and has no CPU "
            "implementation (use the reference's cpsig for host arrays).")


class PathInput:
    def __init__(self, path, time_aug, lead_lag, end_time, name="path"):
        check_array(path, name)
        self.path = own_contiguous(path)
        check_dtype(self.path, name)
        if self.path.ndim < 2:
            raise ValueError(name + " must have at least rank 2, got rank " + str(self.path.ndim) + ".")
        self.batch_shape = tuple(self.path.shape[:-2])
        self.batch_size = prod(self.batch_shape) if self.batch_shape else 1
        self.data_length = self.path.shape[-2]
        self.data_dimension = self.path.shape[-1]
        if self.data_dimension == 0:
            raise ValueError(name + " has 0 channels (dimension). Path dimension must be at least 1.")
        _require_gpu(self.path, name)
        self.type_ = "torch"
        self.dtype = str(self.path.dtype)[6:]
        self.device = self.path.device
        self.data_ptr = cast(self.path.data_ptr(), POINTER(DTYPES[self.dtype]))
        self.time_aug, self.lead_lag, self.end_time = time_aug, lead_lag, end_time
        self.length = 2 * self.data_length - 1 if lead_lag else self.data_length
        self.dimension = (2 * self.data_dimension if lead_lag else self.data_dimension) + (1 if time_aug else 0)


class SigInput:
    """A signature-shaped input; a leading column is dropped when the input is one wider than expected."""

    def __init__(self, sig, sig_len, name):
        check_array(sig, name)
        self.sig = own_contiguous(sig)
        check_dtype(self.sig, name)
        if self.sig.ndim < 1:
            raise ValueError(name + " must have at least rank 1, got rank 0.")
        self.batch_shape = tuple(self.sig.shape[:-1])
        self.batch_size = prod(self.batch_shape) if self.batch_shape else 1
        length = self.sig.shape[-1]
        if length == sig_len + 1:
            self.sig = own_contiguous(self.sig[..., 1:])
            length = sig_len
        if length != sig_len:
            raise ValueError(name + " is of incorrect length. Expected " + str(sig_len) + ", got " + str(length))
        self.type_ = "numpy" if isinstance(self.sig, np.ndarray) else "torch"
        self.dtype = str(self.sig.dtype) if self.type_ == "numpy" else str(self.sig.dtype)[6:]
        _require_gpu(self.sig, name)
        self.device = self.sig.device
        self.data_ptr = cast(self.sig.data_ptr(), POINTER(DTYPES[self.dtype]))


def empty_like_input(data, shape):
    dtype = torch.float32 if data.dtype == "float32" else torch.float64
    out = torch.empty((*data.batch_shape, *shape), dtype=dtype, device=data.device)
    return out, cast(out.data_ptr(), POINTER(DTYPES[data.dtype]))


class on_device:
    """``with on_device(dev):`` makes ``dev`` the current device for the C call; free when it already is."""

    def __init__(self, device):
        self.idx = device.index if device.index is not None else torch.cuda.current_device()
        self.prev = None

    def __enter__(self):
        cur = torch.cuda.current_device()
        if cur != self.idx:
            self.prev = cur
            torch.cuda.set_device(self.idx)
        return self

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False
