"""MI355X-native batched truncated path signatures (forward and backward).

Drop-in for ``pysiglib.sig`` / ``pysiglib.sig_backprop`` / ``pysiglib.torch_api.sig`` on GPU tensors.
"""
from . import torch_api
from .coef import extract_sig_coef, sig_coef, sig_coef_backprop, word_to_idx
from .log_sig import clear_cache, log_sig, prepare_log_sig, sig_to_log_sig, sig_to_log_sig_backprop
from .ops import (linear_sig, sig_combine, sig_combine_backprop, sig_join, sig_join_backprop, transform_path,
                  transform_path_backprop)
from .sig import sig, sig_backprop, signature
from .sig_length import log_sig_length, sig_length

__all__ = ["sig", "signature", "sig_backprop", "sig_length", "sig_combine", "sig_combine_backprop", "sig_join",
           "sig_join_backprop", "linear_sig", "transform_path", "transform_path_backprop", "sig_coef", "sig_coef_backprop",
           "extract_sig_coef", "word_to_idx", "log_sig", "sig_to_log_sig", "sig_to_log_sig_backprop", "prepare_log_sig", "clear_cache",
           "log_sig_length", "torch_api"]
