"""Pins the oracle's sig_combine / transform_path functions and their backward passes.

Evidence that does not come from the oracle: the reference's hand-computed vectors (tests/_ops_kats.py), its golden
float32 gradients of sig_combine (tests/golden/reference_fixture.npz, keys sig_comb_bp_*), Chen's identity against the
already pinned signature, an independent torch Chen product with autograd, and the textbook lead-lag / time
augmentation written with repeat / linspace.
"""
import numpy as np
import pytest
import torch

from oracle import sigref
from tests import _mathref as M
from tests import _ops_kats as K


def _levels(flat, d, degree):
    out, off = [], 0
    for k in range(1, degree + 1):
        out.append(flat[:, off:off + d ** k])
        off += d ** k
    return out


def _chen_torch(a, b, d, degree):
    """Independent Chen product of (B, S) tensors without scalar term."""
    return torch.cat(M._chen(_levels(a, d, degree), _levels(b, d, degree), degree), dim=1)


def test_combine_kats():
    for s1, s2, want, d, deg in K.COMBINE:
        got = sigref.sig_combine(np.array(s1), np.array(s2), d, deg)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-14)
        got = sigref.sig_combine(np.array(s1[1:]), np.array(s2[1:]), d, deg)
        np.testing.assert_allclose(got, want[1:], rtol=0, atol=1e-14)


@pytest.mark.parametrize("d,deg", [(2, 5), (5, 4), (3, 1), (1, 6), (7, 3)])
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-10), (np.float32, 1e-4)])
def test_combine_is_chen_identity(d, deg, dtype, tol):
    if d == 1 and dtype == np.float32:
        pytest.skip("x^k/k! of a small net increment is ill-conditioned in float32")
    rng = np.random.default_rng(d * 31 + deg)
    x = rng.uniform(size=(6, 25, d)).astype(dtype)
    s1 = sigref.signature(x[:, :11], deg)
    s2 = sigref.signature(x[:, 10:], deg)
    whole = sigref.signature(x, deg)
    got = sigref.sig_combine(s1, s2, d, deg)
    assert got.dtype == dtype
    assert np.max(M.level_rel_err(got, whole, d, deg)) < tol
    # scalar-term format in, scalar-term format out
    one = np.ones((6, 1), dtype=dtype)
    got1 = sigref.sig_combine(np.hstack([one, s1]), np.hstack([one, s2]), d, deg)
    assert np.all(got1[:, 0] == 1)
    np.testing.assert_array_equal(got1[:, 1:], got)


@pytest.mark.parametrize("d,deg", [(2, 4), (3, 3), (4, 2)])
def test_combine_vs_independent_product_on_arbitrary_tensors(d, deg):
    # not group-like: catches a transposed operand, which Chen's identity on signatures of similar paths may not
    rng = np.random.default_rng(5)
    n = sigref.sig_length(d, deg) - 1
    a, b = rng.standard_normal((4, n)), rng.standard_normal((4, n))
    want = _chen_torch(torch.tensor(a), torch.tensor(b), d, deg).numpy()
    np.testing.assert_allclose(sigref.sig_combine(a, b, d, deg), want, rtol=1e-13, atol=1e-13)


def test_combine_backprop_kats():
    for g, s1, s2, w1, w2, d, deg in K.COMBINE_BACKPROP:
        d1, d2 = sigref.sig_combine_backprop(np.array(g), np.array(s1), np.array(s2), d, deg)
        np.testing.assert_allclose(d1, w1, rtol=0, atol=1e-14)
        np.testing.assert_allclose(d2, w2, rtol=0, atol=1e-14)
    # as one batch
    g, s1, s2, w1, w2 = (np.array([k[i] for k in K.COMBINE_BACKPROP]) for i in range(5))
    d1, d2 = sigref.sig_combine_backprop(g, s1, s2, 2, 2)
    np.testing.assert_allclose(d1, w1, rtol=0, atol=1e-14)
    np.testing.assert_allclose(d2, w2, rtol=0, atol=1e-14)


@pytest.mark.parametrize("deg", range(1, 6))
def test_combine_backprop_golden(fixtures, deg):
    # tolerance of the reference's own test (tests/test_sig_combine_backprop.py:24): the expected values are float32
    s1, s2, g = (fixtures["sig_comb_bp_%s__d%d" % (k, deg)] for k in ("sig1", "sig2", "derivs"))
    d1, d2 = sigref.sig_combine_backprop(g, s1, s2, 3, deg)
    np.testing.assert_allclose(d1[:, 1:], fixtures["sig_comb_bp_d1__d%d" % deg], rtol=0, atol=1e-5)
    np.testing.assert_allclose(d2[:, 1:], fixtures["sig_comb_bp_d2__d%d" % deg], rtol=0, atol=1e-5)
    assert np.all(d1[:, 0] == 0) and np.all(d2[:, 0] == 0)


@pytest.mark.parametrize("d,deg", [(2, 5), (3, 4), (5, 2), (1, 4), (4, 1)])
def test_combine_backprop_vs_autograd(d, deg):
    rng = np.random.default_rng(17 * d + deg)
    n = sigref.sig_length(d, deg) - 1
    a, b, g = (rng.standard_normal((3, n)) for _ in range(3))
    ta, tb = torch.tensor(a, requires_grad=True), torch.tensor(b, requires_grad=True)
    _chen_torch(ta, tb, d, deg).backward(torch.tensor(g))
    d1, d2 = sigref.sig_combine_backprop(g, a, b, d, deg)
    np.testing.assert_allclose(d1, ta.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(d2, tb.grad.numpy(), rtol=1e-12, atol=1e-12)
    # float32 instance
    d1f, d2f = sigref.sig_combine_backprop(g.astype(np.float32), a.astype(np.float32), b.astype(np.float32), d, deg)
    assert d1f.dtype == np.float32
    np.testing.assert_allclose(d1f, ta.grad.numpy(), rtol=2e-4, atol=2e-4)
    np.testing.assert_allclose(d2f, tb.grad.numpy(), rtol=2e-4, atol=2e-4)


def test_transform_kats():
    for path, kw, want in K.TRANSFORM:
        got = sigref.transform_path(np.array(path), **kw)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-15)


@pytest.mark.parametrize("kw", [dict(time_aug=True), dict(lead_lag=True), dict(time_aug=True, lead_lag=True),
                                dict(time_aug=True, end_time=2.5), dict(time_aug=True, lead_lag=True, end_time=.3)])
@pytest.mark.parametrize("shape", [(3, 2, 1), (2, 9, 4), (1, 100, 5)])
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-13), (np.float32, 1e-5)])
def test_transform_vs_textbook(kw, shape, dtype, tol):
    rng = np.random.default_rng(3)
    x = rng.uniform(size=shape).astype(dtype)
    want = M.augment(torch.tensor(x), **kw).numpy()
    got = sigref.transform_path(x, **kw)
    assert got.dtype == dtype and got.shape == want.shape
    np.testing.assert_allclose(got, want, rtol=0, atol=tol)


def test_transform_feeds_signature():
    # sig(transform_path(x)) == sig(x, augmentation flags): ties the materialised transform to the on-the-fly one
    rng = np.random.default_rng(9)
    x = rng.uniform(size=(4, 12, 2))
    for kw in (dict(time_aug=True, end_time=1.5), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)):
        a = sigref.signature(sigref.transform_path(x, **kw), 4)
        b = sigref.signature(x, 4, **kw)
        np.testing.assert_allclose(a, b, rtol=1e-12, atol=1e-12)


def test_transform_backprop_kats():
    for g, kw, want in K.TRANSFORM_BACKPROP:
        got = sigref.transform_path_backprop(g, want.shape[1], want.shape[0], **kw)
        np.testing.assert_allclose(got, want, rtol=0, atol=1e-14)


@pytest.mark.parametrize("kw", [dict(time_aug=True), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)])
@pytest.mark.parametrize("shape", [(2, 2, 3), (3, 7, 2), (1, 1, 4)])
def test_transform_backprop_vs_autograd(kw, shape):
    if kw.get("time_aug") and shape[1] < 2:
        pytest.skip("time augmentation needs two points")
    rng = np.random.default_rng(11)
    x = torch.tensor(rng.uniform(size=shape), requires_grad=True)
    y = M.augment(x, **kw)
    g = rng.standard_normal(tuple(y.shape))
    y.backward(torch.tensor(g))
    got = sigref.transform_path_backprop(g, shape[2], shape[1], **kw)
    np.testing.assert_allclose(got, x.grad.numpy(), rtol=1e-13, atol=1e-13)
    gotf = sigref.transform_path_backprop(g.astype(np.float32), shape[2], shape[1], **kw)
    np.testing.assert_allclose(gotf, x.grad.numpy(), rtol=1e-5, atol=1e-5)
