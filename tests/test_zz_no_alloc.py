"""The entry point that allocates nothing (cusig_amd_sig_backprop_noalloc_d) against sig_backprop_cuda_d, through the
C ABI: same gradients (float64, <= 1e-10 of the largest entry per path), on calls in a row that share the built-in
scratch array, the later ones smaller than the first; and a clear refusal of shapes beyond that array.

The yardstick here is the allocating entry point, not the oracle: sig_backprop_cuda_d runs the same kernel families and
is itself checked against the oracle in tests/test_gpu_parity.py.  What this file adds is the property the entry point
exists for: a call neither takes nor returns device memory (free device memory and the library's workspace pool are
the same before and after), and a refused call touches nothing."""
import ctypes

import numpy as np
import pytest

torch = pytest.importorskip("torch")

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _ptr(t):
    return ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_double))


def _both(L, rng, batch, length, dim, degree, time_aug=False, lead_lag=False, scalar=False, stream=None):
    x = torch.tensor(rng.standard_normal((batch, length, dim)) * 0.5, device=DEV)
    d_aug = (2 * dim if lead_lag else dim) + (1 if time_aug else 0)
    n = int(L.CUSIG.cusig_amd_sig_length(d_aug, degree)) - (0 if scalar else 1)
    sig = torch.empty((batch, n), dtype=torch.float64, device=DEV)
    rc = L.CUSIG_SIGNATURE["float64"](_ptr(x), _ptr(sig), batch, dim, length, degree, time_aug, lead_lag, 1.5, True, scalar,
                                      None, 0, 0, 0)
    assert rc == 0, L.last_error_message()
    g = torch.tensor(rng.standard_normal((batch, n)), device=DEV)
    ref = torch.full_like(x, float("nan"))
    rc = L.CUSIG_SIG_BACKPROP["float64"](_ptr(x), _ptr(ref), _ptr(g), _ptr(sig), batch, dim, length, degree, time_aug,
                                         lead_lag, 1.5, scalar, None, 0, 0, 0)
    assert rc == 0, L.last_error_message()
    out = torch.full_like(x, float("nan"))
    torch.cuda.synchronize()
    handle = stream.cuda_stream if stream is not None else None
    if stream is not None:
        stream.wait_stream(torch.cuda.current_stream())
    # the first call of a kernel may make the runtime load its code object: measure on the second
    for attempt in range(2):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        pool_before = int(L.CUSIG.cusig_amd_workspace_bytes())
        rc = L.CUSIG_SIG_BACKPROP_NOALLOC(_ptr(x), _ptr(out), _ptr(g), _ptr(sig), batch, dim, length, degree, time_aug,
                                          lead_lag, 1.5, scalar, handle)
        assert rc == 0, L.last_error_message()
        torch.cuda.synchronize()       # the call only enqueues
        if attempt:
            assert torch.cuda.mem_get_info()[0] == free_before, "the call changed the free device memory"
            assert int(L.CUSIG.cusig_amd_workspace_bytes()) == pool_before, "the call grew the workspace pool"
    ref, out = ref.cpu().numpy(), out.cpu().numpy()
    assert np.isfinite(out).all()
    scale = np.abs(ref).reshape(batch, -1).max(axis=1)
    err = (np.abs(out - ref).reshape(batch, -1).max(axis=1) / np.maximum(scale, 1e-300)).max()
    assert err <= 1e-10, (batch, length, dim, degree, err)


def test_no_alloc_backward_matches_the_allocating_entry_point():
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_workspace_bytes.argtypes = ()
    L.CUSIG.cusig_amd_workspace_bytes.restype = ctypes.c_uint64
    rng = np.random.default_rng(77)
    assert int(L.CUSIG.cusig_amd_noalloc_scratch_bytes()) == 32 << 20
    # two calls in a row on the shared scratch array, the second smaller; then other kernel families
    _both(L, rng, 8, 200, 10, 5)
    _both(L, rng, 3, 50, 4, 3)
    _both(L, rng, 5, 33, 3, 4, time_aug=True, lead_lag=True, scalar=True)     # lead-lag-aware sweep
    _both(L, rng, 4, 70, 20, 2)                                                 # degree 2: closed form on the matrix cores
    _both(L, rng, 2, 9, 3, 1)                                                   # degree 1: endpoints only
    _both(L, rng, 3, 40, 23, 3)                                                 # run-time-dimension kernel
    _both(L, rng, 6, 120, 6, 4, stream=torch.cuda.Stream())                     # on a stream of the caller's
    _both(L, rng, 2, 30, 2, 6)


def test_no_alloc_backward_refuses_what_does_not_fit():
    from pysiglib_amd import _loader as L
    x = torch.zeros(8, dtype=torch.float64, device=DEV)
    out = torch.full((8,), float("nan"), dtype=torch.float64, device=DEV)
    # 4096 paths x 2000 points x 8 channels: increments and their gradient need ~1 GB; rejected before any launch
    rc = L.CUSIG_SIG_BACKPROP_NOALLOC(_ptr(x), _ptr(out), _ptr(x), _ptr(x), 4096, 8, 2000, 3, False, False, 1.0, False, None)
    assert rc == 2
    assert "scratch" in L.last_error_message()
    torch.cuda.synchronize()
    assert bool(torch.isnan(out).all()), "a refused call wrote to its output"
    rc = L.CUSIG_SIG_BACKPROP_NOALLOC(_ptr(x), _ptr(x), _ptr(x), _ptr(x), 1, 0, 5, 3, False, False, 1.0, False, None)
    assert rc == 2      # dimension 0, as in sig_backprop_cuda_d
    torch.cuda.synchronize()
