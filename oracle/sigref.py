"""ctypes binding of the CPU oracle ``libsigref.so`` (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's CPU-baseline leg may import this
module; the shipped package never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsigref.so")


def build(force=False):
    """Compile the oracle with the Makefile beside this file."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, capture_output=True)
    subprocess.run(["make", "-C", _HERE], check=True, capture_output=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    u64, i32 = ctypes.c_uint64, ctypes.c_int
    lib.sigref_sig_length.restype = u64
    lib.sigref_sig_length.argtypes = (u64, u64)
    lib.sigref_max_threads.restype = i32
    for suf, real in (("f", ctypes.c_float), ("d", ctypes.c_double)):
        ptr = ctypes.POINTER(real)
        f = getattr(lib, "sigref_signature_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, u64, u64, u64, u64, i32, i32, real, i32, i32, i32)
        g = getattr(lib, "sigref_sig_backprop_" + suf)
        g.restype = i32
        g.argtypes = (ptr, ptr, ptr, ptr, u64, u64, u64, u64, i32, i32, real, i32, i32)
        f = getattr(lib, "sigref_sig_combine_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, u64, u64, u64, i32)
        f = getattr(lib, "sigref_sig_combine_backprop_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, ptr, ptr, u64, u64, u64, i32)
        f = getattr(lib, "sigref_transform_path_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, u64, u64, u64, i32, i32, real)
        f = getattr(lib, "sigref_transform_path_backprop_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, u64, u64, u64, i32, i32)
        pu = ctypes.POINTER(u64)
        f = getattr(lib, "sigref_sig_coef_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, pu, u64, pu, u64, u64, u64, i32, i32, real, i32)
        f = getattr(lib, "sigref_sig_coef_backprop_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, ptr, pu, u64, pu, u64, u64, u64, i32, i32, real)
        f = getattr(lib, "sigref_sig_to_log_sig_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, u64, u64, u64, i32)
        f = getattr(lib, "sigref_sig_to_log_sig_backprop_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, u64, u64, u64, i32)
        f = getattr(lib, "sigref_linear_sig_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, u64, u64, u64, i32)
        f = getattr(lib, "sigref_sig_join_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, u64, u64, u64, i32, i32)
        f = getattr(lib, "sigref_sig_join_backprop_" + suf)
        f.restype = i32
        f.argtypes = (ptr, ptr, ptr, ptr, ptr, u64, u64, u64, i32, i32)
    return lib


LIB = _load()


def max_threads():
    return int(LIB.sigref_max_threads())


def sig_length(dimension, degree):
    return int(LIB.sigref_sig_length(dimension, degree))


def _suffix(dtype):
    if dtype == np.float32:
        return "f", ctypes.c_float
    if dtype == np.float64:
        return "d", ctypes.c_double
    raise TypeError("oracle supports float32 and float64 only")


def _aug_dim(d, time_aug, lead_lag):
    return (2 * d if lead_lag else d) + (1 if time_aug else 0)


def signature(path, degree, time_aug=False, lead_lag=False, end_time=1.0, horner=True,
              scalar_term=False, n_jobs=1):
    """Oracle forward pass. ``path`` is (B, len, d) or (len, d), float32/float64."""
    path = np.ascontiguousarray(path)
    single = path.ndim == 2
    if single:
        path = path[None]
    batch, length, dim = path.shape
    suf, real = _suffix(path.dtype)
    n = sig_length(_aug_dim(dim, time_aug, lead_lag), degree) - (0 if scalar_term else 1)
    out = np.empty((batch, n), dtype=path.dtype)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_signature_" + suf)(
        path.ctypes.data_as(ptr), out.ctypes.data_as(ptr), batch, dim, length, degree,
        int(time_aug), int(lead_lag), float(end_time), int(horner), int(scalar_term), n_jobs)
    if rc:
        raise RuntimeError("sigref_signature returned %d" % rc)
    return out[0] if single else out


def sig_backprop(path, sig, sig_derivs, degree, time_aug=False, lead_lag=False, end_time=1.0,
                 n_jobs=1):
    """Oracle backward pass; scalar_term is inferred from the width of ``sig``."""
    path = np.ascontiguousarray(path)
    single = path.ndim == 2
    if single:
        path, sig, sig_derivs = path[None], np.asarray(sig)[None], np.asarray(sig_derivs)[None]
    batch, length, dim = path.shape
    suf, real = _suffix(path.dtype)
    full = sig_length(_aug_dim(dim, time_aug, lead_lag), degree)
    sig = np.ascontiguousarray(sig, dtype=path.dtype)
    sig_derivs = np.ascontiguousarray(sig_derivs, dtype=path.dtype)
    if sig.shape[-1] == full:
        scalar_term = True
    elif sig.shape[-1] == full - 1:
        scalar_term = False
    else:
        raise ValueError("sig has the wrong width")
    if sig_derivs.shape != sig.shape:
        raise ValueError("sig_derivs and sig must have the same shape")
    out = np.empty_like(path)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_backprop_" + suf)(
        path.ctypes.data_as(ptr), out.ctypes.data_as(ptr), sig_derivs.ctypes.data_as(ptr),
        sig.ctypes.data_as(ptr), batch, dim, length, degree, int(time_aug), int(lead_lag),
        float(end_time), int(scalar_term), n_jobs)
    if rc:
        raise RuntimeError("sigref_sig_backprop returned %d" % rc)
    return out[0] if single else out


def _rows(arr, dtype):
    a = np.ascontiguousarray(arr, dtype=dtype)
    return a.reshape(-1, a.shape[-1])


def sig_combine(sig1, sig2, dimension, degree):
    """Oracle Chen product; scalar_term is inferred from the width."""
    sig1 = np.asarray(sig1)
    suf, real = _suffix(sig1.dtype)
    a, b = _rows(sig1, sig1.dtype), _rows(sig2, sig1.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    out = np.empty_like(a)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_combine_" + suf)(a.ctypes.data_as(ptr), b.ctypes.data_as(ptr), out.ctypes.data_as(ptr),
                                                   a.shape[0], dimension, degree, int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_combine returned %d" % rc)
    return out.reshape(sig1.shape)


def sig_combine_backprop(derivs, sig1, sig2, dimension, degree):
    sig1 = np.asarray(sig1)
    suf, real = _suffix(sig1.dtype)
    a, b, g = _rows(sig1, sig1.dtype), _rows(sig2, sig1.dtype), _rows(derivs, sig1.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    d1, d2 = np.empty_like(a), np.empty_like(a)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_combine_backprop_" + suf)(
        g.ctypes.data_as(ptr), d1.ctypes.data_as(ptr), d2.ctypes.data_as(ptr), a.ctypes.data_as(ptr),
        b.ctypes.data_as(ptr), a.shape[0], dimension, degree, int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_combine_backprop returned %d" % rc)
    return d1.reshape(sig1.shape), d2.reshape(sig1.shape)


def transform_path(path, time_aug=False, lead_lag=False, end_time=1.0):
    path = np.ascontiguousarray(path)
    single = path.ndim == 2
    if single:
        path = path[None]
    batch, length, dim = path.shape
    suf, real = _suffix(path.dtype)
    out = np.empty((batch, 2 * length - 1 if lead_lag else length, _aug_dim(dim, time_aug, lead_lag)), dtype=path.dtype)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_transform_path_" + suf)(path.ctypes.data_as(ptr), out.ctypes.data_as(ptr), batch, dim,
                                                      length, int(time_aug), int(lead_lag), float(end_time))
    if rc:
        raise RuntimeError("sigref_transform_path returned %d" % rc)
    return out[0] if single else out


def transform_path_backprop(derivs, dimension, length, time_aug=False, lead_lag=False):
    derivs = np.ascontiguousarray(derivs)
    single = derivs.ndim == 2
    if single:
        derivs = derivs[None]
    suf, real = _suffix(derivs.dtype)
    out = np.empty((derivs.shape[0], length, dimension), dtype=derivs.dtype)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_transform_path_backprop_" + suf)(derivs.ctypes.data_as(ptr), out.ctypes.data_as(ptr),
                                                               derivs.shape[0], dimension, length, int(time_aug),
                                                               int(lead_lag))
    if rc:
        raise RuntimeError("sigref_transform_path_backprop returned %d" % rc)
    return out[0] if single else out


def linear_sig(displacement, dimension, degree, scalar_term=False):
    """Oracle signature of straight-line displacements (..., dimension)."""
    disp = np.ascontiguousarray(displacement)
    suf, real = _suffix(disp.dtype)
    z = _rows(disp, disp.dtype)
    n = sig_length(dimension, degree) - (0 if scalar_term else 1)
    out = np.empty((z.shape[0], n), dtype=disp.dtype)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_linear_sig_" + suf)(z.ctypes.data_as(ptr), out.ctypes.data_as(ptr), z.shape[0], dimension,
                                                  degree, int(scalar_term))
    if rc:
        raise RuntimeError("sigref_linear_sig returned %d" % rc)
    return out.reshape(disp.shape[:-1] + (n,))


def sig_join(sig, displacement, dimension, degree, prepend=False):
    sig = np.asarray(sig)
    suf, real = _suffix(sig.dtype)
    a, z = _rows(sig, sig.dtype), _rows(displacement, sig.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    out = np.empty_like(a)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_join_" + suf)(a.ctypes.data_as(ptr), z.ctypes.data_as(ptr), out.ctypes.data_as(ptr),
                                                a.shape[0], dimension, degree, int(prepend), int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_join returned %d" % rc)
    return out.reshape(sig.shape)


def sig_join_backprop(derivs, sig, displacement, dimension, degree, prepend=False):
    sig = np.asarray(sig)
    suf, real = _suffix(sig.dtype)
    a, z, g = _rows(sig, sig.dtype), _rows(displacement, sig.dtype), _rows(derivs, sig.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    dsig, dz = np.empty_like(a), np.empty_like(z)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_join_backprop_" + suf)(
        g.ctypes.data_as(ptr), dsig.ctypes.data_as(ptr), dz.ctypes.data_as(ptr), a.ctypes.data_as(ptr),
        z.ctypes.data_as(ptr), a.shape[0], dimension, degree, int(prepend), int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_join_backprop returned %d" % rc)
    return dsig.reshape(sig.shape), dz.reshape(np.shape(displacement))


def _words(words):
    flat = np.array([i for w in words for i in w], dtype=np.uint64)
    degs = np.array([len(w) for w in words], dtype=np.uint64)
    if flat.size == 0:
        flat = np.zeros(1, dtype=np.uint64)
    return flat, degs


def sig_coef(path, words, time_aug=False, lead_lag=False, end_time=1.0, prefixes=False):
    """Oracle coefficients of the given words (list of tuples) for path (length, dim) or (batch, length, dim)."""
    path = np.ascontiguousarray(path)
    single = path.ndim == 2
    if single:
        path = path[None]
    batch, length, dim = path.shape
    suf, real = _suffix(path.dtype)
    flat, degs = _words(words)
    row = sum((max(len(w), 1) if prefixes else 1) for w in words)
    out = np.empty((batch, row), dtype=path.dtype)
    ptr, pu = ctypes.POINTER(real), ctypes.POINTER(ctypes.c_uint64)
    rc = getattr(LIB, "sigref_sig_coef_" + suf)(path.ctypes.data_as(ptr), out.ctypes.data_as(ptr), flat.ctypes.data_as(pu),
                                                len(words), degs.ctypes.data_as(pu), batch, dim, length, int(time_aug),
                                                int(lead_lag), float(end_time), int(prefixes))
    if rc:
        raise RuntimeError("sigref_sig_coef returned %d" % rc)
    return out[0] if single else out


def sig_coef_backprop(path, words, coefs, derivs, time_aug=False, lead_lag=False, end_time=1.0):
    """coefs / derivs in the prefixes=True layout."""
    path = np.ascontiguousarray(path)
    single = path.ndim == 2
    if single:
        path = path[None]
    batch, length, dim = path.shape
    suf, real = _suffix(path.dtype)
    flat, degs = _words(words)
    c = np.ascontiguousarray(coefs, dtype=path.dtype).reshape(batch, -1)
    g = np.ascontiguousarray(derivs, dtype=path.dtype).reshape(batch, -1)
    out = np.zeros_like(path)
    ptr, pu = ctypes.POINTER(real), ctypes.POINTER(ctypes.c_uint64)
    rc = getattr(LIB, "sigref_sig_coef_backprop_" + suf)(
        path.ctypes.data_as(ptr), out.ctypes.data_as(ptr), c.ctypes.data_as(ptr), g.ctypes.data_as(ptr),
        flat.ctypes.data_as(pu), len(words), degs.ctypes.data_as(pu), batch, dim, length, int(time_aug), int(lead_lag),
        float(end_time))
    if rc:
        raise RuntimeError("sigref_sig_coef_backprop returned %d" % rc)
    return out[0] if single else out


def sig_to_log_sig(sig, dimension, degree, method=0):
    """Oracle log signature; ``dimension`` is the augmented dimension.  method 0: expanded (same width as ``sig``);
    1: its coefficients at the Lyndon words; 2: coordinates in the Lyndon basis (oracle/lyndon.py)."""
    if method:
        from . import lyndon
        full = sig_to_log_sig(sig, dimension, degree, 0)
        off = 1 if np.asarray(sig).shape[-1] == sig_length(dimension, degree) else 0
        return np.ascontiguousarray(lyndon.compress(full[..., off:], dimension, degree, method))
    sig = np.asarray(sig)
    suf, real = _suffix(sig.dtype)
    a = _rows(sig, sig.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    out = np.empty_like(a)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_to_log_sig_" + suf)(a.ctypes.data_as(ptr), out.ctypes.data_as(ptr), a.shape[0], dimension,
                                                      degree, int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_to_log_sig returned %d" % rc)
    return out.reshape(sig.shape)


def sig_to_log_sig_backprop(sig, derivs, dimension, degree, method=0):
    if method:
        from . import lyndon
        expanded = lyndon.compress_backprop(derivs, dimension, degree, method)
        if np.asarray(sig).shape[-1] == sig_length(dimension, degree):
            expanded = np.concatenate([np.zeros(expanded.shape[:-1] + (1,), dtype=expanded.dtype), expanded], axis=-1)
        return sig_to_log_sig_backprop(sig, np.ascontiguousarray(expanded), dimension, degree, 0)
    sig = np.asarray(sig)
    suf, real = _suffix(sig.dtype)
    a, g = _rows(sig, sig.dtype), _rows(derivs, sig.dtype)
    scalar_term = a.shape[1] == sig_length(dimension, degree)
    out = np.empty_like(a)
    ptr = ctypes.POINTER(real)
    rc = getattr(LIB, "sigref_sig_to_log_sig_backprop_" + suf)(a.ctypes.data_as(ptr), out.ctypes.data_as(ptr),
                                                               g.ctypes.data_as(ptr), a.shape[0], dimension, degree,
                                                               int(scalar_term))
    if rc:
        raise RuntimeError("sigref_sig_to_log_sig_backprop returned %d" % rc)
    return out.reshape(sig.shape)
