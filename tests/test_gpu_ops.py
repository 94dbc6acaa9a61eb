"""Parity of sig_combine / transform_path and their backward passes (HIP, through the C ABI) with the CPU oracle,
the reference's hand-computed vectors and its golden float32 gradients.

Tolerances: float64 1e-10, float32 1e-4 (relative to the per-level / per-row max norm); exact for the pure copies
of transform_path; golden float32 gradients at the reference's 1e-5 (tests/test_sig_combine_backprop.py:24).
"""
import ctypes

import numpy as np
import pytest
import torch

from tests import _ops_kats as K
from tests._mathref import level_rel_err

pytestmark = pytest.mark.gpu

TOL = {np.float64: 1e-10, np.float32: 1e-4}
DEV = "cuda:0"


@pytest.fixture(scope="module")
def P():
    import pysiglib_amd
    assert torch.cuda.is_available()
    return pysiglib_amd


@pytest.fixture(scope="module")
def oracle():
    from oracle import sigref
    return sigref


@pytest.fixture(params=[0, 1], ids=["adjoint-auto", "adjoint-streaming"])
def chen_mode(request):
    """Kernels of the Chen product's adjoint: automatic choice, then the streaming kernels forced onto every shape."""
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_chen_adjoint.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_chen_adjoint.restype = None
    L.CUSIG.cusig_amd_force_chen_adjoint(request.param)
    yield request.param
    L.CUSIG.cusig_amd_force_chen_adjoint(0)


@pytest.fixture(params=[1, 2], ids=["low-auto", "low-lds"])
def chen_low(request):
    """Chen product kernels (sig_combine, tensor logarithm): automatic choice, then the factors' short levels kept in LDS
    for every shape and element type."""
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_chen_low_levels.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_chen_low_levels.restype = None
    L.CUSIG.cusig_amd_set_chen_low_levels(request.param)
    yield request.param
    L.CUSIG.cusig_amd_set_chen_low_levels(1)


def dev(a, dtype=None):
    return torch.tensor(np.ascontiguousarray(a, dtype=dtype), device=DEV)


def row_rel_err(got, ref):
    got = got.reshape(-1, ref.shape[-1]).astype(np.float64)
    ref = ref.reshape(-1, ref.shape[-1]).astype(np.float64)
    den = np.maximum(np.abs(ref).max(axis=1), np.finfo(np.float64).tiny)
    return float((np.abs(got - ref).max(axis=1) / den).max())


def test_combine_kats(P):
    for s1, s2, want, d, deg in K.COMBINE:
        got = P.sig_combine(dev(s1), dev(s2), d, deg)
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=0, atol=1e-14)
        got = P.sig_combine(dev(s1[1:]), dev(s2[1:]), d, deg)
        np.testing.assert_allclose(got.cpu().numpy(), want[1:], rtol=0, atol=1e-14)


@pytest.mark.parametrize("d,deg,batch", [(2, 5, 7), (5, 4, 33), (3, 1, 4), (1, 6, 3), (7, 3, 130), (10, 5, 32),
                                         (37, 2, 5), (2, 14, 2), (4, 4, 9), (6, 3, 5), (11, 3, 3), (13, 3, 5), (9, 4, 2)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_combine_vs_oracle(P, oracle, chen_low, d, deg, batch, dtype, scalar_term):
    rng = np.random.default_rng(100 * d + deg)
    n = oracle.sig_length(d, deg) - 1
    scale = np.concatenate([np.full(d ** k, 1.0 / np.sqrt(float(d) ** k)) for k in range(1, deg + 1)])
    a = (rng.standard_normal((batch, n)) * scale).astype(dtype)
    b = (rng.standard_normal((batch, n)) * scale).astype(dtype)
    if scalar_term:
        one = np.ones((batch, 1), dtype=dtype)
        a, b = np.hstack([one, a]), np.hstack([one, b])
    want = oracle.sig_combine(a, b, d, deg)
    got = P.sig_combine(dev(a), dev(b), d, deg).cpu().numpy()
    assert got.shape == want.shape and got.dtype == dtype
    off = 1 if scalar_term else 0
    if scalar_term:
        assert np.all(got[:, 0] == 1)
    assert np.max(level_rel_err(got[:, off:], want[:, off:], d, deg)) < TOL[dtype]


@pytest.mark.parametrize("deg", range(1, 6))
def test_combine_chen_identity(P, deg):
    # the reference's own test of sig_combine (tests/test_sig_combine.py:27-54)
    rng = np.random.default_rng(42 + deg)
    x1 = rng.uniform(size=(32, 100, 5))
    x2 = rng.uniform(size=(32, 100, 5))
    whole = P.sig(dev(np.concatenate([x1, x2], axis=1)), deg)
    s1 = P.sig(dev(x1), deg)
    s2 = P.sig(dev(np.concatenate([x1[:, -1:], x2], axis=1)), deg)
    got = P.sig_combine(s1, s2, 5, deg)
    assert got.device.type == "cuda"
    np.testing.assert_allclose(got.cpu().numpy(), whole.cpu().numpy(), rtol=0, atol=1e-10)


def test_combine_batch_shapes_views_and_errors(P, oracle):
    d, deg = 10, 3
    n = P.sig_length(d, deg)
    col = torch.rand((32, 1), dtype=torch.float64, device=DEV)
    view = col.expand(-1, n)                      # stride-0 view, as in the reference's non-contiguous test
    np.testing.assert_array_equal(P.sig_combine(view, view, d, deg).cpu().numpy(),
                                  P.sig_combine(view.clone(), view.clone(), d, deg).cpu().numpy())
    a = torch.rand((2, 3, n), dtype=torch.float64, device=DEV)
    b = torch.rand((2, 3, n), dtype=torch.float64, device=DEV)
    got = P.sig_combine(a, b, d, deg)
    assert got.shape == (2, 3, n)
    np.testing.assert_allclose(got.cpu().numpy(), oracle.sig_combine(a.cpu().numpy(), b.cpu().numpy(), d, deg),
                               rtol=1e-12, atol=1e-12)
    assert P.sig_combine(a[0, 0], b[0, 0], d, deg).shape == (n,)
    empty = torch.empty((0, n), dtype=torch.float64, device=DEV)
    assert P.sig_combine(empty, empty, d, deg).shape == (0, n)
    with pytest.raises(ValueError):
        P.sig_combine(a, b[..., :-1], d, deg)
    with pytest.raises(ValueError):
        P.sig_combine(a, b[0], d, deg)
    with pytest.raises(ValueError):
        P.sig_combine(a, b.float(), d, deg)
    with pytest.raises(RuntimeError):
        P.sig_combine(a.cpu(), b.cpu(), d, deg)
    with pytest.raises(TypeError):
        P.sig_combine(a, b, 10.0, deg)


def test_combine_backprop_kats(P):
    for g, s1, s2, w1, w2, d, deg in K.COMBINE_BACKPROP:
        d1, d2 = P.sig_combine_backprop(dev(g), dev(s1), dev(s2), d, deg)
        np.testing.assert_allclose(d1.cpu().numpy(), w1, rtol=0, atol=1e-14)
        np.testing.assert_allclose(d2.cpu().numpy(), w2, rtol=0, atol=1e-14)
    g, s1, s2, w1, w2 = (np.array([k[i] for k in K.COMBINE_BACKPROP]) for i in range(5))
    d1, d2 = P.sig_combine_backprop(dev(g), dev(s1), dev(s2), 2, 2)
    np.testing.assert_allclose(d1.cpu().numpy(), w1, rtol=0, atol=1e-14)
    np.testing.assert_allclose(d2.cpu().numpy(), w2, rtol=0, atol=1e-14)


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_combine_backprop_golden(P, fixtures, deg, dtype):
    s1, s2, g = (dev(fixtures["sig_comb_bp_%s__d%d" % (k, deg)], dtype) for k in ("sig1", "sig2", "derivs"))
    d1, d2 = P.sig_combine_backprop(g, s1, s2, 3, deg)
    atol = 1e-5 if dtype == np.float64 else 1e-4
    np.testing.assert_allclose(d1.cpu().numpy()[:, 1:], fixtures["sig_comb_bp_d1__d%d" % deg], rtol=0, atol=atol)
    np.testing.assert_allclose(d2.cpu().numpy()[:, 1:], fixtures["sig_comb_bp_d2__d%d" % deg], rtol=0, atol=atol)
    assert torch.all(d1[:, 0] == 0) and torch.all(d2[:, 0] == 0)
    one1, one2 = P.sig_combine_backprop(g[0], s1[0], s2[0], 3, deg)
    # long sums are cut into parts that are added with atomics: equal up to the order of the additions
    np.testing.assert_allclose(one1.cpu().numpy(), d1[0].cpu().numpy(), rtol=1e-6 if dtype == np.float32 else 1e-14, atol=atol * 1e-6)
    np.testing.assert_allclose(one2.cpu().numpy(), d2[0].cpu().numpy(), rtol=1e-6 if dtype == np.float32 else 1e-14, atol=atol * 1e-6)


@pytest.mark.parametrize("d,deg,batch", [(2, 5, 7), (5, 4, 33), (3, 1, 4), (1, 6, 3), (7, 3, 130), (10, 5, 32),
                                         (37, 2, 5), (2, 14, 2), (4, 4, 9), (6, 3, 5), (11, 3, 3), (13, 3, 5), (9, 4, 2)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_combine_backprop_vs_oracle(P, oracle, chen_mode, d, deg, batch, dtype, scalar_term):
    rng = np.random.default_rng(7 * d + deg)
    n = oracle.sig_length(d, deg) - (0 if scalar_term else 1)
    a, b, g = (rng.standard_normal((batch, n)).astype(dtype) for _ in range(3))
    if scalar_term:
        a[:, 0] = 1
        b[:, 0] = 1
    w1, w2 = oracle.sig_combine_backprop(g, a, b, d, deg)
    d1, d2 = P.sig_combine_backprop(dev(g), dev(a), dev(b), d, deg)
    assert d1.shape == w1.shape and d2.shape == w2.shape
    assert row_rel_err(d1.cpu().numpy(), w1) < TOL[dtype]
    assert row_rel_err(d2.cpu().numpy(), w2) < TOL[dtype]


@pytest.mark.parametrize("d,deg,batch", [(2, 20, 1), (3, 12, 2), (4, 10, 1), (6, 8, 1), (12, 6, 1), (33, 4, 1), (100, 3, 2)])
def test_combine_backprop_long_rows(P, oracle, d, deg, batch):
    """Rows of 0.8-3.3 million coefficients: the streaming adjoint kernels with several levels of words above a
    block's own (deep signatures of few channels) and the wide-path kernel (more than 32 channels)."""
    rng = np.random.default_rng(11 * d + deg)
    n = oracle.sig_length(d, deg) - 1
    scale = np.concatenate([np.full(d ** k, 1.0 / np.sqrt(float(d) ** k)) for k in range(1, deg + 1)])
    a, b, g = (rng.standard_normal((batch, n)) * scale for _ in range(3))
    w1, w2 = oracle.sig_combine_backprop(g, a, b, d, deg)
    d1, d2 = P.sig_combine_backprop(dev(g), dev(a), dev(b), d, deg)
    assert row_rel_err(d1.cpu().numpy(), w1) < TOL[np.float64]
    assert row_rel_err(d2.cpu().numpy(), w2) < TOL[np.float64]


def test_combine_autograd(P):
    d, deg = 3, 4
    n = P.sig_length(d, deg)
    a = torch.rand((5, n), dtype=torch.float64, device=DEV, requires_grad=True)
    b = torch.rand((5, n), dtype=torch.float64, device=DEV, requires_grad=True)
    w = torch.rand((5, n), dtype=torch.float64, device=DEV)
    (P.torch_api.sig_combine(a, b, d, deg) * w).sum().backward()
    d1, d2 = P.sig_combine_backprop(w, a.detach(), b.detach(), d, deg)
    np.testing.assert_allclose(a.grad.cpu().numpy(), d1.cpu().numpy(), rtol=1e-14, atol=1e-14)
    np.testing.assert_allclose(b.grad.cpu().numpy(), d2.cpu().numpy(), rtol=1e-14, atol=1e-14)
    # directional derivative: <w, C(a + h u, b) - C(a - h u, b)> / 2h == <dA, u>  (the product is bilinear: exact up to rounding)
    u = torch.rand_like(w)
    h = 1e-3
    num = ((P.sig_combine(a.detach() + h * u, b.detach(), d, deg) - P.sig_combine(a.detach() - h * u, b.detach(), d, deg))
           * w).sum() / (2 * h)
    assert abs(float(num) - float((d1 * u).sum())) < 1e-8 * max(1.0, abs(float(num)))


def test_transform_kats(P):
    for path, kw, want in K.TRANSFORM:
        got = P.transform_path(dev(path), **kw)
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=0, atol=1e-15)
    for g, kw, want in K.TRANSFORM_BACKPROP:
        got = P.transform_path_backprop(dev(g), **kw)
        assert got.shape == want.shape
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=0, atol=1e-14)


@pytest.mark.parametrize("kw", [dict(time_aug=True), dict(lead_lag=True), dict(time_aug=True, lead_lag=True),
                                dict(time_aug=True, end_time=2.5), dict(time_aug=True, lead_lag=True, end_time=.3)])
@pytest.mark.parametrize("shape", [(3, 2, 1), (2, 9, 4), (10, 100, 5), (1, 3, 70), (300, 33, 3)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_transform_vs_oracle(P, oracle, kw, shape, dtype):
    rng = np.random.default_rng(shape[1])
    x = rng.uniform(size=shape).astype(dtype)
    want = oracle.transform_path(x, **kw)
    got = P.transform_path(dev(x), **kw).cpu().numpy()
    assert got.shape == want.shape and got.dtype == dtype
    nt = -1 if kw.get("time_aug") else None
    np.testing.assert_array_equal(got[..., :nt], want[..., :nt])                 # copied channels: bit-exact
    if nt:
        np.testing.assert_allclose(got[..., -1], want[..., -1], rtol=0, atol=TOL[dtype] * kw.get("end_time", 1.0))
    g = rng.standard_normal(want.shape).astype(dtype)
    wantg = oracle.transform_path_backprop(g, shape[2], shape[1], time_aug=kw.get("time_aug", False),
                                           lead_lag=kw.get("lead_lag", False))
    gotg = P.transform_path_backprop(dev(g), **kw).cpu().numpy()
    assert gotg.shape == wantg.shape
    np.testing.assert_allclose(gotg, wantg, rtol=0, atol=TOL[dtype] * 4)


def test_transform_feeds_signature_and_autograd(P):
    rng = np.random.default_rng(5)
    x = dev(rng.uniform(size=(6, 20, 3)))
    for kw in (dict(time_aug=True, end_time=1.5), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)):
        a = P.sig(P.transform_path(x, **kw), 4)
        b = P.sig(x, 4, **kw)
        np.testing.assert_allclose(a.cpu().numpy(), b.cpu().numpy(), rtol=1e-11, atol=1e-11)
        xr = x.clone().requires_grad_(True)
        y = P.torch_api.transform_path(xr, **kw)
        w = torch.rand_like(y)
        (y * w).sum().backward()
        np.testing.assert_array_equal(xr.grad.cpu().numpy(), P.transform_path_backprop(w, **kw).cpu().numpy())


def test_transform_identity_batch_shapes_and_errors(P):
    x = torch.rand((2, 3, 8, 4), dtype=torch.float64, device=DEV)
    assert P.transform_path(x) is x
    assert P.transform_path_backprop(x) is x
    y = P.transform_path(x, time_aug=True, lead_lag=True)
    assert y.shape == (2, 3, 15, 9)
    np.testing.assert_array_equal(y[1, 2].cpu().numpy(), P.transform_path(x[1, 2], time_aug=True, lead_lag=True).cpu().numpy())
    assert P.transform_path_backprop(y, time_aug=True, lead_lag=True).shape == x.shape
    assert P.transform_path(x[:, :, ::2], lead_lag=True).shape == (2, 3, 7, 8)          # strided view
    empty = torch.empty((0, 8, 4), dtype=torch.float64, device=DEV)
    assert P.transform_path(empty, time_aug=True).shape == (0, 8, 5)
    one = torch.rand((1, 4), dtype=torch.float64, device=DEV)
    assert P.transform_path(one, lead_lag=True).shape == (1, 8)
    with pytest.raises(ValueError):
        P.transform_path(one, time_aug=True)
    with pytest.raises(ValueError):
        P.transform_path_backprop(torch.rand((4, 6), dtype=torch.float64, device=DEV), lead_lag=True)
    with pytest.raises(TypeError):
        P.transform_path(x, time_aug=True, end_time=1)
    with pytest.raises(RuntimeError):
        P.transform_path(x.cpu(), time_aug=True)


@pytest.mark.parametrize("d,deg,batch", [(2, 6, 5), (3, 4, 70), (5, 3, 4), (1, 7, 3), (4, 1, 2), (3, 0, 3), (10, 5, 32),
                                         (40, 2, 3), (2, 14, 2)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_linear_sig_vs_oracle(P, oracle, d, deg, batch, dtype, scalar_term):
    rng = np.random.default_rng(13 * d + deg)
    z = rng.standard_normal((batch, d)).astype(dtype)
    want = oracle.linear_sig(z, d, deg, scalar_term=scalar_term)
    got = P.linear_sig(dev(z), d, deg, scalar_term=scalar_term).cpu().numpy()
    assert got.shape == want.shape and got.dtype == dtype
    if want.shape[1]:
        assert row_rel_err(got, want) < TOL[dtype]
    if scalar_term:
        assert np.all(got[:, 0] == 1)
    if deg >= 1 and not scalar_term:        # equals the signature of the two-point path, computed by the sweep kernels
        x = np.zeros((batch, 2, d), dtype=dtype)
        x[:, 1] = z
        np.testing.assert_allclose(got, P.sig(dev(x), deg).cpu().numpy(), rtol=0, atol=TOL[dtype] * max(1.0, np.abs(want).max()))


@pytest.mark.parametrize("d,deg,batch", [(2, 5, 5), (3, 4, 70), (5, 2, 4), (1, 5, 3), (4, 1, 2), (10, 5, 32), (40, 2, 3),
                                         (2, 14, 2), (3, 7, 4), (2, 19, 1), (7, 3, 9), (13, 3, 5)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("prepend", [False, True])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_sig_join_vs_oracle(P, oracle, chen_mode, chen_low, d, deg, batch, dtype, prepend, scalar_term):
    rng = np.random.default_rng(5 * d + deg)
    n = oracle.sig_length(d, deg) - 1
    scale = np.concatenate([np.full(d ** k, 1.0 / np.sqrt(float(d) ** k)) for k in range(1, deg + 1)])
    a = (rng.standard_normal((batch, n)) * scale).astype(dtype)
    z = (rng.standard_normal((batch, d)) * 0.7).astype(dtype)
    g = rng.standard_normal((batch, n)).astype(dtype)
    if scalar_term:
        a = np.hstack([np.ones((batch, 1), dtype=dtype), a])
        g = np.hstack([np.full((batch, 1), 2.0, dtype=dtype), g])
    off = 1 if scalar_term else 0
    want = oracle.sig_join(a, z, d, deg, prepend=prepend)
    got = P.sig_join(dev(a), dev(z), d, deg, prepend=prepend).cpu().numpy()
    assert got.shape == want.shape and got.dtype == dtype
    assert np.max(level_rel_err(got[:, off:], want[:, off:], d, deg)) < TOL[dtype]
    if scalar_term:
        assert np.all(got[:, 0] == 1)
    ws, wz = oracle.sig_join_backprop(g, a, z, d, deg, prepend=prepend)
    ds, dz = P.sig_join_backprop(dev(g), dev(a), dev(z), d, deg, prepend=prepend)
    assert ds.shape == ws.shape and dz.shape == wz.shape
    assert row_rel_err(ds.cpu().numpy(), ws) < TOL[dtype]
    assert row_rel_err(dz.cpu().numpy(), wz) < (TOL[dtype] if dtype == np.float64 else 5e-4)
    if scalar_term:
        assert torch.all(ds[:, 0] == 0)


@pytest.mark.parametrize("prepend", [False, True])
def test_sig_join_extends_the_path_and_autograd(P, prepend):
    rng = np.random.default_rng(77)
    d, deg = 4, 4
    x = rng.uniform(size=(6, 30, d))
    z = rng.standard_normal((6, d))
    longer = np.concatenate([x[:, :1] - z[:, None], x], axis=1) if prepend else np.concatenate([x, x[:, -1:] + z[:, None]], axis=1)
    s = P.sig(dev(x), deg)
    got = P.sig_join(s, dev(z), d, deg, prepend=prepend)
    np.testing.assert_allclose(got.cpu().numpy(), P.sig(dev(longer), deg).cpu().numpy(), rtol=1e-10, atol=1e-12)
    e = P.linear_sig(dev(z), d, deg)
    comb = P.sig_combine(e, s, d, deg) if prepend else P.sig_combine(s, e, d, deg)
    np.testing.assert_allclose(got.cpu().numpy(), comb.cpu().numpy(), rtol=1e-12, atol=1e-13)
    sr, zr = s.clone().requires_grad_(True), dev(z).requires_grad_(True)
    w = torch.rand_like(s)
    (P.torch_api.sig_join(sr, zr, d, deg, prepend=prepend) * w).sum().backward()
    ds, dz = P.sig_join_backprop(w, s, dev(z), d, deg, prepend=prepend)
    np.testing.assert_allclose(sr.grad.cpu().numpy(), ds.cpu().numpy(), rtol=1e-14, atol=1e-14)
    # the displacement gradient is accumulated with atomics: equal up to the order of the additions
    np.testing.assert_allclose(zr.grad.cpu().numpy(), dz.cpu().numpy(), rtol=1e-13, atol=1e-13)


def test_join_linear_batch_shapes_and_errors(P, oracle):
    d, deg = 3, 3
    n = P.sig_length(d, deg)
    s = torch.rand((2, 4, n), dtype=torch.float64, device=DEV)
    z = torch.rand((2, 4, d), dtype=torch.float64, device=DEV)
    out = P.sig_join(s, z, d, deg)
    assert out.shape == (2, 4, n)
    np.testing.assert_allclose(out.cpu().numpy(), oracle.sig_join(s.cpu().numpy(), z.cpu().numpy(), d, deg), rtol=1e-12, atol=1e-12)
    assert P.sig_join(s[0, 0], z[0, 0], d, deg).shape == (n,)
    assert P.linear_sig(z, d, deg).shape == (2, 4, n)
    assert P.linear_sig(z[1, 2], d, deg, scalar_term=True).shape == (n + 1,)
    ds, dz = P.sig_join_backprop(out, s, z, d, deg)
    assert ds.shape == s.shape and dz.shape == z.shape
    empty_s = torch.empty((0, n), dtype=torch.float64, device=DEV)
    empty_z = torch.empty((0, d), dtype=torch.float64, device=DEV)
    assert P.sig_join(empty_s, empty_z, d, deg).shape == (0, n)
    assert P.linear_sig(empty_z, d, deg).shape == (0, n)
    with pytest.raises(ValueError):
        P.sig_join(s, z[0], d, deg)
    with pytest.raises(ValueError):
        P.sig_join(s, z.float(), d, deg)
    with pytest.raises(ValueError):
        P.sig_join(s, z[..., :2], d, deg)
    with pytest.raises(ValueError):
        P.linear_sig(z, d + 1, deg)
    with pytest.raises(RuntimeError):
        P.linear_sig(z.cpu(), d, deg)


def test_wide_index_arithmetic(P, oracle):
    """The 64-bit index path of the coefficient-per-thread kernels (rows of 2^31 coefficients or more in production),
    forced here on small shapes; also covers the time-segmented forward's Chen fold."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_wide_index.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_wide_index.restype = None
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_segments.restype = None
    rng = np.random.default_rng(31)
    d, deg, batch = 3, 6, 9
    n = oracle.sig_length(d, deg) - 1
    a, b, g = (rng.standard_normal((batch, n)) * 0.3 for _ in range(3))
    z = rng.standard_normal((batch, d))
    x = rng.uniform(size=(4, 9, 2))
    L.CUSIG.cusig_amd_force_wide_index(1)
    try:
        np.testing.assert_allclose(P.sig_combine(dev(a), dev(b), d, deg).cpu().numpy(), oracle.sig_combine(a, b, d, deg),
                                   rtol=1e-12, atol=1e-12)
        d1, d2 = P.sig_combine_backprop(dev(g), dev(a), dev(b), d, deg)
        w1, w2 = oracle.sig_combine_backprop(g, a, b, d, deg)
        np.testing.assert_allclose(d1.cpu().numpy(), w1, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(d2.cpu().numpy(), w2, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(P.linear_sig(dev(z), d, deg).cpu().numpy(), oracle.linear_sig(z, d, deg), rtol=1e-12, atol=1e-12)
        for prepend in (False, True):
            np.testing.assert_allclose(P.sig_join(dev(a), dev(z), d, deg, prepend=prepend).cpu().numpy(),
                                       oracle.sig_join(a, z, d, deg, prepend=prepend), rtol=1e-12, atol=1e-12)
            ds, dz = P.sig_join_backprop(dev(g), dev(a), dev(z), d, deg, prepend=prepend)
            ws, wz = oracle.sig_join_backprop(g, a, z, d, deg, prepend=prepend)
            np.testing.assert_allclose(ds.cpu().numpy(), ws, rtol=1e-12, atol=1e-12)
            np.testing.assert_allclose(dz.cpu().numpy(), wz, rtol=1e-11, atol=1e-11)
        kw = dict(time_aug=True, lead_lag=True, end_time=2.0)
        y = P.transform_path(dev(x), **kw)
        np.testing.assert_allclose(y.cpu().numpy(), oracle.transform_path(x, **kw), rtol=0, atol=1e-14)
        gy = rng.standard_normal(tuple(y.shape))
        np.testing.assert_allclose(P.transform_path_backprop(dev(gy), **kw).cpu().numpy(),
                                   oracle.transform_path_backprop(gy, 2, 9, time_aug=True, lead_lag=True), rtol=0, atol=1e-13)
        L.CUSIG.cusig_amd_force_segments(3)
        xs = rng.uniform(size=(2, 200, 3))
        np.testing.assert_allclose(P.sig(dev(xs), 4).cpu().numpy(), oracle.signature(xs, 4), rtol=1e-10, atol=1e-12)
    finally:
        L.CUSIG.cusig_amd_force_segments(0)
        L.CUSIG.cusig_amd_force_wide_index(0)


# ---------------------------------------------------------------------------
# sig_coef / sig_coef_backprop
# ---------------------------------------------------------------------------
def _all_words(d, degree):
    import itertools
    return [w for k in range(1, degree + 1) for w in itertools.product(range(d), repeat=k)]


def test_sig_coef_trivial_cases(P):
    x = torch.tensor([[0., 0.], [1., 1.]], device=DEV)
    np.testing.assert_array_equal(P.sig_coef(x, [(0,), (1,)]).cpu().numpy(), [1., 1.])
    np.testing.assert_array_equal(P.sig_coef(x[None], [(0,), (1,)]).cpu().numpy(), [[1., 1.]])
    np.testing.assert_array_equal(P.sig_coef(x[:1], [(0,), (1,)]).cpu().numpy(), [0., 0.])
    np.testing.assert_array_equal(P.sig_coef(x, [(), (0, 1)], prefixes=True).cpu().numpy(), [1., 1., 0.5])
    np.testing.assert_array_equal(P.sig_coef(x, (1, 0)).cpu().numpy(), [0.5])


@pytest.mark.parametrize("aug", [{}, dict(time_aug=True, end_time=1.5), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("shape", [(3, 15, 2), (70, 40, 3), (1, 2, 5)])
def test_sig_coef_vs_oracle(P, oracle, aug, dtype, shape):
    rng = np.random.default_rng(shape[0] + shape[1])
    x = rng.uniform(size=shape).astype(dtype)
    d = shape[2]
    da = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    words = [(da - 1,), (0, da - 1), (1, 0, 1, da - 1), (), (da - 1, da - 1, 0), (0, 0), (0, 1, 0, 1, 0, 1, 1),
             tuple(i % da for i in range(12)), tuple((3 * i + 1) % da for i in range(20))]
    for prefixes in (False, True):
        want = oracle.sig_coef(x, words, prefixes=prefixes, **aug)
        got = P.sig_coef(dev(x), words, prefixes=prefixes, **aug).cpu().numpy()
        assert got.shape == want.shape and got.dtype == dtype
        if dtype == np.float64:
            np.testing.assert_allclose(got, want, rtol=1e-10, atol=1e-13)
        else:       # tiny high-degree coefficients cancel in float32: measured against the largest entry of the row
            assert bwd_err(got, want) < TOL[dtype]
    cp = oracle.sig_coef(x, words, prefixes=True, **aug)
    g = rng.standard_normal(cp.shape).astype(dtype)
    want = oracle.sig_coef_backprop(x, words, cp, g, **aug)
    got = P.sig_coef_backprop(dev(x), words, dev(cp), dev(g), **aug).cpu().numpy()
    assert got.shape == x.shape
    assert bwd_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("shape", [(2, 9, 300), (2, 6, 2000), (2, 6, 2800), (1, 5, 5000), (3, 200, 12)])
def test_sig_coef_wide_and_long_paths(P, oracle, dtype, shape):
    """Paths too wide for the LDS staging of the points (forward) or of the per-channel sums (backward) take the
    kernels that read and add straight from / to memory; a long narrow path crosses several chunks of steps."""
    rng = np.random.default_rng(shape[1] + shape[2])
    x = (rng.uniform(size=shape) * 0.5).astype(dtype)
    d = shape[2]
    words = [(d - 1,), (0, d - 1), (d // 2, 1, d - 1), (), (d - 1, d - 1, 0), (1, 0, 1, d - 2)] + \
            [tuple(int(v) for v in rng.integers(0, d, size=3)) for _ in range(70)]
    cp = oracle.sig_coef(x, words, prefixes=True)
    got = P.sig_coef(dev(x), words, prefixes=True).cpu().numpy()
    assert bwd_err(got, cp) < TOL[dtype]
    g = rng.standard_normal(cp.shape).astype(dtype)
    want = oracle.sig_coef_backprop(x, words, cp, g)
    got = P.sig_coef_backprop(dev(x), words, dev(cp), dev(g)).cpu().numpy()
    assert got.shape == x.shape
    assert bwd_err(got, want) < TOL[dtype]


def bwd_err(got, ref):
    got = got.reshape(ref.shape[0], -1).astype(np.float64)
    ref = ref.reshape(ref.shape[0], -1).astype(np.float64)
    den = np.maximum(np.abs(ref).max(axis=1), np.finfo(np.float64).tiny)
    return float((np.abs(got - ref).max(axis=1) / den).max())


@pytest.mark.parametrize("kw", [{}, dict(time_aug=True), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)])
def test_sig_coef_full_word_set_is_the_signature(P, kw):
    # the reference's own test of sig_coef (tests/test_sig_coef.py:114-163)
    rng = np.random.default_rng(3)
    x = dev(rng.uniform(size=(10, 100, 2)))
    da = (4 if kw.get("lead_lag") else 2) + (1 if kw.get("time_aug") else 0)
    deg = 4
    words = _all_words(da, deg)
    sig = P.sig(x, deg, **kw)
    np.testing.assert_allclose(P.sig_coef(x, words, **kw).cpu().numpy(), sig.cpu().numpy(), rtol=1e-10, atol=1e-13)
    np.testing.assert_array_equal(P.extract_sig_coef(sig, words, 2, **kw).cpu().numpy(), sig.cpu().numpy())
    one = P.extract_sig_coef(P.sig(x, deg, scalar_term=True, **kw), [(da - 1, 0)], 2, scalar_term=True, **kw)
    np.testing.assert_array_equal(one.cpu().numpy()[:, 0], sig.cpu().numpy()[:, P.word_to_idx((da - 1, 0), da, deg)])


def test_sig_coef_autograd_and_batch_shapes(P, oracle):
    rng = np.random.default_rng(12)
    words = [(2, 0, 1), (1, 1), (), (0,)]
    x = dev(rng.uniform(size=(2, 3, 9, 3)))
    xr = x.clone().requires_grad_(True)
    out = P.torch_api.sig_coef(xr, words, time_aug=True, end_time=0.5)
    assert out.shape == (2, 3, 4)
    w = torch.rand_like(out)
    (out * w).sum().backward()
    # gradient of the selected coefficients == backprop with the weight on each word's last prefix
    cp = P.sig_coef(x, words, prefixes=True, time_aug=True, end_time=0.5)
    assert cp.shape == (2, 3, 7)
    g = torch.zeros_like(cp)
    g[..., [2, 4, 5, 6]] = w
    want = oracle.sig_coef_backprop(x.cpu().numpy().reshape(6, 9, 3), words, cp.cpu().numpy().reshape(6, 7),
                                    g.cpu().numpy().reshape(6, 7), time_aug=True, end_time=0.5)
    np.testing.assert_allclose(xr.grad.cpu().numpy().reshape(6, 9, 3), want, rtol=1e-11, atol=1e-12)
    pre = P.torch_api.sig_coef(x, words, prefixes=True, time_aug=True, end_time=0.5)
    np.testing.assert_array_equal(pre.cpu().numpy(), cp.cpu().numpy())
    assert P.sig_coef(x[0, 0], (0, 1)).shape == (1,)
    empty = torch.empty((0, 9, 3), dtype=torch.float64, device=DEV)
    assert P.sig_coef(empty, words).shape == (0, 4)
    assert P.sig_coef_backprop(empty, words, torch.empty((0, 7), dtype=torch.float64, device=DEV),
                               torch.empty((0, 7), dtype=torch.float64, device=DEV)).shape == (0, 9, 3)
    with pytest.raises(ValueError):
        P.sig_coef(x, [(3,)])
    with pytest.raises(ValueError):
        P.sig_coef(x, [])
    with pytest.raises(TypeError):
        P.sig_coef(x, [[0, 1]])
    with pytest.raises(ValueError):
        P.sig_coef_backprop(x, words, cp[..., :-1], g[..., :-1])
    with pytest.raises(RuntimeError):
        P.sig_coef(x.cpu(), words)
    with pytest.raises(Exception, match="not implemented"):
        P.sig_coef(x, [(0,) * 65])


def test_sig_coef_abi_rejects_bad_letters(P):
    import ctypes
    from pysiglib_amd import _loader as L
    x = torch.rand((2, 5, 3), dtype=torch.float64, device=DEV)
    out = torch.empty((2, 1), dtype=torch.float64, device=DEV)
    letters = torch.tensor([0, 3], dtype=torch.int64, device=DEV)       # 3 is out of range for 3 channels
    degrees = torch.tensor([2], dtype=torch.int64, device=DEV)
    pd = lambda t: ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_double))
    pu = lambda t: ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_uint64))
    assert L.CUSIG_SIG_COEF["float64"](pd(x), pd(out), pu(letters), 1, pu(degrees), 2, 3, 5, False) == 2
    assert "out of range" in L.last_error_message()
    assert L.CUSIG_SIG_COEF["float64"](pd(x), pd(out), pu(letters), 1, pu(degrees), 2, 0, 5, False) == 2


# ---------------------------------------------------------------------------
# sig_to_log_sig / log_sig (method 0)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_log_sig_golden(P, fixtures, deg, dtype):
    # the reference's own tests of the expanded log signature (tests/test_log_sig.py:101-144)
    x = dev(fixtures["path"].astype(dtype))
    tol = TOL[dtype]
    np.testing.assert_allclose(P.log_sig(x, deg, method=0).cpu().numpy(), fixtures["logsig_exp__d%d" % deg], rtol=0, atol=tol)
    np.testing.assert_allclose(P.log_sig(x[0], deg, method=0).cpu().numpy(), fixtures["logsig_exp__d%d" % deg][0], rtol=0, atol=tol)
    np.testing.assert_allclose(P.log_sig(x, deg, time_aug=True, method=0).cpu().numpy(), fixtures["logsig_exp_ta__d%d" % deg],
                               rtol=0, atol=tol)
    if deg <= 4:
        np.testing.assert_allclose(P.log_sig(x[:2], deg, lead_lag=True, method=0).cpu().numpy(),
                                   fixtures["logsig_exp_ll__d%d" % deg], rtol=0, atol=tol)


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_log_sig_backprop_golden(P, fixtures, deg, dtype):
    # tests/test_log_sig_backprop.py:49-100 of the reference: path gradient through log_sig(method=0)
    for key, kw in (("logsig_bp_exp", {}), ("logsig_bp_exp_ta", dict(time_aug=True))):
        x = torch.tensor(fixtures["path"], dtype=dtype, device=DEV, requires_grad=True)
        ls = P.torch_api.log_sig(x, deg, method=0, **kw)
        ls.backward(torch.tensor(fixtures["%s_derivs__d%d" % (key, deg)], dtype=dtype, device=DEV))
        np.testing.assert_allclose(x.grad.cpu().numpy(), fixtures["%s_expected__d%d" % (key, deg)], rtol=0,
                                   atol=1e-5 if dtype == torch.float64 else 1e-4)


@pytest.mark.parametrize("d,deg,batch", [(2, 6, 5), (3, 4, 70), (5, 3, 4), (1, 5, 3), (4, 1, 2), (3, 0, 3), (10, 5, 32),
                                         (40, 2, 3), (2, 12, 2), (6, 4, 3), (13, 3, 2)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_sig_to_log_sig_vs_oracle(P, oracle, chen_mode, chen_low, d, deg, batch, dtype, scalar_term):
    rng = np.random.default_rng(3 * d + deg)
    n = oracle.sig_length(d, deg) - 1
    scale = np.concatenate([np.full(d ** k, 0.5 / np.sqrt(float(d) ** k)) for k in range(1, deg + 1)]) if deg else np.zeros(0)
    a = (rng.standard_normal((batch, n)) * scale).astype(dtype)
    g = rng.standard_normal((batch, n)).astype(dtype)
    if scalar_term:
        a = np.hstack([np.ones((batch, 1), dtype=dtype), a])
        g = np.hstack([np.full((batch, 1), 3.0, dtype=dtype), g])
    elif deg == 0:
        pytest.skip("empty rows")
    off = 1 if scalar_term else 0
    want = oracle.sig_to_log_sig(a, d, deg)
    got = P.sig_to_log_sig(dev(a), d, deg, method=0).cpu().numpy()
    assert got.shape == want.shape and got.dtype == dtype
    if scalar_term:
        assert np.all(got[:, 0] == 0)
    if deg:
        assert np.max(level_rel_err(got[:, off:], want[:, off:], d, deg)) < TOL[dtype]
    wantb = oracle.sig_to_log_sig_backprop(a, g, d, deg)
    gotb = P.sig_to_log_sig_backprop(dev(a), dev(g), d, deg, method=0).cpu().numpy()
    assert gotb.shape == wantb.shape
    if scalar_term:
        assert np.all(gotb[:, 0] == 0)
    if deg:
        assert row_rel_err(gotb[:, off:], wantb[:, off:]) < TOL[dtype] * (1 if dtype == np.float64 else 10)


@pytest.mark.parametrize("method", [0, 1, 2])
def test_sig_to_log_sig_out_of_memory_halves_the_batch(P, method):
    """A workspace the device cannot hold (forced from the host) makes sig_to_log_sig and its backward retry on halves
    of the batch, like the reference's launchers (siglib/cusig/cu_runtime_utils.h:103-105,212-235): same results as the
    undisturbed call, rows of either form (expanded, Lyndon coordinates) at their own stride."""
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_alloc_limit.argtypes = (ctypes.c_uint64,)
    L.CUSIG.cusig_amd_set_alloc_limit.restype = None
    L.CUSIG.cusig_amd_alloc_retries.restype = ctypes.c_int
    d, deg, batch = 4, 5, 48
    rng = np.random.default_rng(91 + method)
    x = np.cumsum(rng.standard_normal((batch, 12, d)), axis=1) * 0.3
    sig = P.sig(dev(x), deg)
    if method:
        P.prepare_log_sig(d, deg, method)
    want = P.sig_to_log_sig(sig, d, deg, method=method)
    g = dev(rng.standard_normal(tuple(want.shape)))
    wantb = P.sig_to_log_sig_backprop(sig, g, d, deg, method=method)
    row_bytes = sig.shape[1] * 8
    try:
        L.CUSIG.cusig_shutdown()                     # grown workspaces would hide the limit
        if method:
            P.prepare_log_sig(d, deg, method)        # (the shutdown dropped the prepared tables)
        before = L.CUSIG.cusig_amd_alloc_retries()
        L.CUSIG.cusig_amd_set_alloc_limit(batch * row_bytes)         # the forward wants two rows per path: half the batch fits
        got = P.sig_to_log_sig(sig, d, deg, method=method)
        mid = L.CUSIG.cusig_amd_alloc_retries()
        assert mid >= before + 1
        gotb = P.sig_to_log_sig_backprop(sig, g, d, deg, method=method)
        assert L.CUSIG.cusig_amd_alloc_retries() >= mid + 1
    finally:
        L.CUSIG.cusig_amd_set_alloc_limit(0)
    assert torch.equal(got, want)
    assert torch.equal(gotb, wantb)


def test_log_sig_identities_shapes_and_errors(P):
    rng = np.random.default_rng(6)
    d, deg = 3, 5
    z = dev(rng.standard_normal((2, 4, d)))
    lg = P.sig_to_log_sig(P.linear_sig(z, d, deg), d, deg, method=0)        # log(exp(z)) = z
    assert lg.shape == (2, 4, P.sig_length(d, deg))
    np.testing.assert_allclose(lg[..., :d].cpu().numpy(), z.cpu().numpy(), rtol=0, atol=1e-14)
    np.testing.assert_allclose(lg[..., d:].cpu().numpy(), 0, rtol=0, atol=1e-13)
    x = dev(rng.uniform(size=(3, 20, d)))
    s = P.sig(x, deg, scalar_term=True)
    np.testing.assert_array_equal(P.sig_to_log_sig(s, d, deg, method=0)[:, 1:].cpu().numpy(),
                                  P.log_sig(x, deg, method=0).cpu().numpy())
    sr = s.clone().requires_grad_(True)
    out = P.torch_api.sig_to_log_sig(sr, d, deg, method=0)
    w = torch.rand_like(out)
    (out * w).sum().backward()
    np.testing.assert_allclose(sr.grad.cpu().numpy(), P.sig_to_log_sig_backprop(s, w, d, deg, method=0).cpu().numpy(),
                               rtol=1e-14, atol=1e-14)
    empty = torch.empty((0, P.sig_length(d, deg)), dtype=torch.float64, device=DEV)
    assert P.sig_to_log_sig(empty, d, deg, method=0).shape == empty.shape
    P.clear_cache()
    with pytest.raises(Exception, match="Could not find prepared cache"):
        P.sig_to_log_sig(s, d, deg)                     # the reference's default, method=1, needs prepare_log_sig
    with pytest.raises(NotImplementedError):
        P.log_sig(x, deg, method=3)
    with pytest.raises(ValueError):
        P.sig_to_log_sig(s, d, deg, method=3)
    with pytest.raises(ValueError):
        P.sig_to_log_sig(s, d, deg, method=7)
    with pytest.raises(ValueError):
        P.sig_to_log_sig(s[:, :-2], d, deg, method=0)
    # the C ABI itself reports the unsupported methods with status 10
    import ctypes
    from pysiglib_amd import _loader as L
    pd = lambda t: ctypes.cast(t.data_ptr(), ctypes.POINTER(ctypes.c_double))
    o = torch.empty_like(s)
    assert L.CUSIG_SIG_TO_LOG_SIG["float64"](pd(s), pd(o), 3, d, deg, 1, True) == 5
    assert "prepared cache" in L.last_error_message()
    assert L.CUSIG_SIG_TO_LOG_SIG["float64"](pd(s), pd(o), 3, d, deg, 5, True) == 2
    assert L.CUSIG.prepare_log_sig_cuda(d, deg, 3, False) == 10


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_log_sig_lyndon_golden(P, fixtures, deg, dtype):
    """tests/test_log_sig.py:143-203 and tests/test_log_sig_backprop.py of the reference: signatory's Lyndon-word
    coordinates and iisignature's Lyndon-basis coordinates of the fixture paths, forward and path gradients."""
    tol = 1e-10 if dtype == torch.float64 else 1e-4
    try:
        P.clear_cache()
        x = dev(fixtures["path"]).to(dtype)
        with pytest.raises(Exception, match="Could not find prepared cache"):
            P.log_sig(x, deg, method=1)
        P.prepare_log_sig(3, deg, 1)
        np.testing.assert_allclose(P.log_sig(x, deg, method=1).cpu().numpy(), fixtures["logsig_words__d%d" % deg], rtol=0, atol=tol)
        np.testing.assert_allclose(P.log_sig(x[0], deg).cpu().numpy(), fixtures["logsig_words__d%d" % deg][0], rtol=0, atol=tol)
        with pytest.raises(Exception, match="Could not find prepared cache"):
            P.log_sig(x, deg, method=2)                  # prepared for method 1 only
        P.prepare_log_sig(3, deg, 2)
        np.testing.assert_allclose(P.log_sig(x, deg, method=2).cpu().numpy(), fixtures["logsig_basis__d%d" % deg], rtol=0, atol=tol)
        np.testing.assert_allclose(P.log_sig(x, deg, method=1, scalar_term=True).cpu().numpy(),
                                   fixtures["logsig_words__d%d" % deg], rtol=0, atol=tol)
        for name, method in (("words", 1), ("basis", 2)):
            xr = torch.tensor(fixtures["path"], dtype=dtype, device=DEV, requires_grad=True)
            ls = P.torch_api.log_sig(xr, deg, method=method)
            ls.backward(torch.tensor(fixtures["logsig_bp_%s_derivs__d%d" % (name, deg)], dtype=dtype, device=DEV))
            np.testing.assert_allclose(xr.grad.cpu().numpy(), fixtures["logsig_bp_%s_expected__d%d" % (name, deg)], rtol=0,
                                       atol=1e-5 if dtype == torch.float64 else 1e-4)
    finally:
        P.clear_cache()


@pytest.mark.parametrize("d,deg,batch", [(2, 7, 5), (3, 4, 70), (5, 4, 4), (1, 5, 3), (4, 1, 2), (8, 3, 33), (6, 5, 2), (20, 2, 3)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_sig_to_log_sig_lyndon_vs_oracle(P, oracle, d, deg, batch, dtype, scalar_term):
    rng = np.random.default_rng(5 * d + deg)
    n = oracle.sig_length(d, deg) - 1
    scale = np.concatenate([np.full(d ** k, 0.5 / np.sqrt(float(d) ** k)) for k in range(1, deg + 1)])
    a = (rng.standard_normal((batch, n)) * scale).astype(dtype)       # arbitrary tensors, not group-like
    if scalar_term:
        a = np.hstack([np.ones((batch, 1), dtype=dtype), a])
    m = P.log_sig_length(d, deg)
    g = rng.standard_normal((batch, m)).astype(dtype)
    try:
        P.prepare_log_sig(d, deg, 2)
        for method in (1, 2):
            want = oracle.sig_to_log_sig(a, d, deg, method=method)
            got = P.sig_to_log_sig(dev(a), d, deg, method=method).cpu().numpy()
            assert got.shape == (batch, m) and got.dtype == dtype
            assert row_rel_err(got, want) < TOL[dtype]
            wantb = oracle.sig_to_log_sig_backprop(a, g, d, deg, method=method)
            gotb = P.sig_to_log_sig_backprop(dev(a), dev(g), d, deg, method=method).cpu().numpy()
            assert gotb.shape == wantb.shape
            if scalar_term:
                assert np.all(gotb[:, 0] == 0)
            off = 1 if scalar_term else 0
            assert row_rel_err(gotb[:, off:], wantb[:, off:]) < TOL[dtype] * (1 if dtype == np.float64 else 10)
    finally:
        P.clear_cache()
