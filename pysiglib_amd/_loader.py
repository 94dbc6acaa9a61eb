"""Loads the HIP shared library ``csrc/libcusig.so`` and binds its C ABI.

Mirrors the role of the reference's loader for its GPU plugin
(pysiglib/load_siglib.py:73-130,484-494,647-664): per-dtype function tables for
the two hot entry points, the last-error getter and a shutdown hook at exit.
There is no CPU fallback: if the library is missing, importing this module
raises.
"""
import atexit
import ctypes
import os
from ctypes import POINTER, c_bool, c_char_p, c_double, c_float, c_int, c_uint64

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("PYSIGLIB_AMD_LIB") or os.path.join(_HERE, "csrc", "libcusig.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "pysiglib_amd: %s is missing. Build it first: python -c 'import __graft_entry__ as g; g.build()' "
        "(or `make -C pysiglib_amd/csrc gen all`)." % LIB_PATH)

CUSIG = ctypes.CDLL(LIB_PATH)

CUSIG.cusig_last_error_message.argtypes = ()
CUSIG.cusig_last_error_message.restype = c_char_p
CUSIG.cusig_shutdown.argtypes = ()
CUSIG.cusig_shutdown.restype = None
CUSIG.cusig_amd_sig_length.argtypes = (c_uint64, c_uint64)
CUSIG.cusig_amd_sig_length.restype = c_uint64
CUSIG.prepare_log_sig_cuda.argtypes = (c_uint64, c_uint64, c_int, c_bool)
CUSIG.prepare_log_sig_cuda.restype = c_int
CUSIG.clear_cache_cuda.argtypes = (c_bool,)
CUSIG.clear_cache_cuda.restype = c_int
CUSIG.cusig_amd_last_sig_nonfinite.argtypes = ()
CUSIG.cusig_amd_last_sig_nonfinite.restype = c_int
CUSIG.cusig_amd_set_profiling.argtypes = (c_int,)
CUSIG.cusig_amd_set_profiling.restype = None
CUSIG.cusig_amd_last_segments.argtypes = ()
CUSIG.cusig_amd_last_segments.restype = c_int
CUSIG.cusig_amd_last_kernel_ms.argtypes = ()
CUSIG.cusig_amd_last_kernel_ms.restype = c_float
CUSIG.cusig_amd_last_kernel_name.argtypes = ()
CUSIG.cusig_amd_last_kernel_name.restype = c_char_p
CUSIG.cusig_amd_kernel_choice.argtypes = (c_int, c_int, c_uint64, c_uint64, POINTER(c_int), POINTER(c_int), POINTER(c_int))
CUSIG.cusig_amd_kernel_choice.restype = c_int

DTYPES = {"float32": c_float, "float64": c_double}
_SUFFIX = {"float32": "_f", "float64": "_d"}


def _table(name, argtypes_of):
    table = {}
    for dtype, real in DTYPES.items():
        fn = getattr(CUSIG, name + _SUFFIX[dtype])
        fn.argtypes = argtypes_of(real)
        fn.restype = c_int
        table[dtype] = fn
    return table


CUSIG_SIGNATURE = _table("signature_cuda", lambda r: (
    POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_uint64, c_bool, c_bool, r, c_bool, c_bool,
    POINTER(r), c_uint64, c_uint64, c_uint64))

CUSIG_SIG_BACKPROP = _table("sig_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_uint64, c_bool, c_bool, r,
    c_bool, POINTER(r), c_uint64, c_uint64, c_uint64))


# the variant of sig_backprop_cuda_d that allocates nothing (float64 only): same arguments without the correction,
# plus the stream to enqueue on
CUSIG_SIG_BACKPROP_NOALLOC = CUSIG.cusig_amd_sig_backprop_noalloc_d
CUSIG_SIG_BACKPROP_NOALLOC.argtypes = (
    POINTER(c_double), POINTER(c_double), POINTER(c_double), POINTER(c_double), c_uint64, c_uint64, c_uint64, c_uint64,
    c_bool, c_bool, c_double, c_bool, ctypes.c_void_p)
CUSIG_SIG_BACKPROP_NOALLOC.restype = c_int
CUSIG.cusig_amd_noalloc_scratch_bytes.argtypes = ()
CUSIG.cusig_amd_noalloc_scratch_bytes.restype = c_uint64

CUSIG_SIG_COMBINE = _table("sig_combine_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool))

CUSIG_SIG_COMBINE_BACKPROP = _table("sig_combine_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool))

CUSIG_TRANSFORM_PATH = _table("transform_path_cuda", lambda r: (
    POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool, c_bool, r))

CUSIG_TRANSFORM_PATH_BACKPROP = _table("transform_path_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool, c_bool, r))


CUSIG_LINEAR_SIG = _table("linear_sig_cuda", lambda r: (POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool))

CUSIG_SIG_JOIN = _table("sig_join_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool, c_bool))

CUSIG_SIG_JOIN_BACKPROP = _table("sig_join_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_bool, c_bool))


CUSIG_SIG_COEF = _table("sig_coef_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(c_uint64), c_uint64, POINTER(c_uint64), c_uint64, c_uint64, c_uint64, c_bool))

CUSIG_SIG_COEF_BACKPROP = _table("sig_coef_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), POINTER(r), POINTER(c_uint64), c_uint64, POINTER(c_uint64), c_uint64, c_uint64,
    c_uint64))


CUSIG_SIG_TO_LOG_SIG = _table("sig_to_log_sig_cuda", lambda r: (
    POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_int, c_bool))

CUSIG_SIG_TO_LOG_SIG_BACKPROP = _table("sig_to_log_sig_backprop_cuda", lambda r: (
    POINTER(r), POINTER(r), POINTER(r), c_uint64, c_uint64, c_uint64, c_int, c_bool))


def last_error_message():
    msg = CUSIG.cusig_last_error_message()
    return msg.decode("utf-8", errors="replace") if msg else ""


@atexit.register
def _shutdown():
    try:
        CUSIG.cusig_shutdown()
    except Exception:  # pragma: no cover - interpreter teardown
        pass
