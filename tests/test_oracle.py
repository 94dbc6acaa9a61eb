"""Pins the CPU oracle (oracle/sigref.c) without running the reference.

Each oracle function is checked against evidence that does not come from the
oracle itself:
  * forward Horner / naive sweeps and both augmentations: the reference's own
    third-party (iisignature) golden vectors and its hand-computed KATs;
  * closed forms: straight line, d = 1, Chen's identity, time reversal,
    re-parameterisation, the level-2 shuffle identity;
  * brute force: iterated sums over segment tuples on tiny inputs;
  * backward: the golden float32 gradients, the hand-computed KATs, torch
    autograd through an independent Chen product (with differentiable
    augmentations) and central finite differences;
  * sig_length: the reference's KAT values incl. the overflow case.
"""
import math

import numpy as np
import pytest

from oracle import sigref
from tests import _mathref as M

AUGS = {
    "sig": ({}, "path"),
    "sig_ta": (dict(time_aug=True), "path"),
    "sig_ll": (dict(lead_lag=True), "path_dim2"),
    "sig_ta_ll": (dict(time_aug=True, lead_lag=True), "path_dim2"),
}


def test_sig_length_kats(kats):
    for d, n, expected in kats["sig_length"]:
        assert sigref.sig_length(d, n) == expected


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("key", list(AUGS))
@pytest.mark.parametrize("horner", [True, False])
@pytest.mark.parametrize("n_jobs", [1, -1])
def test_forward_golden(fixtures, deg, key, horner, n_jobs):
    kw, pkey = AUGS[key]
    expected = fixtures[f"{key}__d{deg}"]
    got = sigref.signature(fixtures[pkey], deg, horner=horner, n_jobs=n_jobs, **kw)
    np.testing.assert_allclose(got, expected, rtol=0, atol=1e-10)
    got32 = sigref.signature(fixtures[pkey].astype(np.float32), deg, horner=horner, n_jobs=n_jobs, **kw)
    np.testing.assert_allclose(got32, expected, rtol=0, atol=1e-4)


def test_forward_kats(kats):
    for k in kats["forward"]:
        dt = np.dtype(k["dtype"])
        path = np.array(k["path"], dtype=dt).reshape(k["batch"], k["length"], k["dimension"])
        for horner in (True, False):
            for n_jobs in (1, -1):
                got = sigref.signature(path, k["degree"], time_aug=k["time_aug"], lead_lag=k["lead_lag"],
                                       end_time=k["end_time"], horner=horner, scalar_term=True, n_jobs=n_jobs)
                tol = 1e-12 if dt == np.float64 else 2e-5
                np.testing.assert_allclose(got.ravel(), np.array(k["expected"]), rtol=tol, atol=tol, err_msg=k["name"])


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("n_jobs", [1, -1])
def test_backward_golden(fixtures, deg, n_jobs):
    x = fixtures["path"]
    sig = sigref.signature(x, deg)
    g_full = fixtures[f"sig_bp_derivs__d{deg}"]          # carries the scalar column
    expected = fixtures[f"sig_bp_expected__d{deg}"]      # float32
    got = sigref.sig_backprop(x, sig, g_full[:, 1:], deg, n_jobs=n_jobs)
    np.testing.assert_allclose(got, expected, rtol=0, atol=1e-5)
    sig1 = sigref.signature(x, deg, scalar_term=True)
    got1 = sigref.sig_backprop(x, sig1, g_full, deg, n_jobs=n_jobs)
    np.testing.assert_array_equal(got, got1)


def test_backward_kats(kats):
    for k in kats["backward"]:
        path = np.array(k["path"]).reshape(k["batch"], k["length"], k["dimension"])
        sig = np.array(k["sig"]).reshape(k["batch"], -1)
        g = np.array(k["derivs"]).reshape(k["batch"], -1)
        for n_jobs in (1, -1):
            got = sigref.sig_backprop(path, sig, g, k["degree"], time_aug=k["time_aug"], lead_lag=k["lead_lag"],
                                      end_time=k["end_time"], n_jobs=n_jobs)
            np.testing.assert_allclose(got.ravel(), np.array(k["expected"]), rtol=1e-12, atol=1e-12, err_msg=k["name"])


@pytest.mark.parametrize("d,deg", [(2, 6), (3, 5), (5, 4), (7, 3), (10, 3)])
def test_straight_line(d, deg):
    rng = np.random.default_rng(d * 10 + deg)
    v = rng.standard_normal(d)
    ts = np.sort(rng.uniform(0, 1, 7))
    ts[0], ts[-1] = 0.0, 1.0
    path = ts[:, None] * v[None, :] + rng.standard_normal(d)[None, :]
    got = sigref.signature(path, deg)
    lvl = np.array(1.0)
    off = 0
    for k in range(1, deg + 1):
        lvl = np.multiply.outer(lvl, v) / k
        np.testing.assert_allclose(got[off:off + d ** k], lvl.ravel(), rtol=1e-12, atol=1e-13)
        off += d ** k


def test_dimension_one_closed_form():
    x = np.array([[0.3], [1.0], [-2.0], [0.7]])
    got = sigref.signature(x, 6, scalar_term=True)
    delta = 0.7 - 0.3
    np.testing.assert_allclose(got, [delta ** k / math.factorial(k) for k in range(7)], rtol=1e-14)


@pytest.mark.parametrize("d,deg,n", [(2, 4, 4), (3, 3, 3), (2, 5, 3)])
def test_brute_force_iterated_sums(d, deg, n):
    rng = np.random.default_rng(100 + d + deg)
    x = rng.standard_normal((n + 1, d))
    np.testing.assert_allclose(sigref.signature(x, deg), M.iterated_sums(x, deg), rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(sigref.signature(x, deg, horner=False), M.iterated_sums(x, deg), rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("d,deg,length", [(2, 5, 12), (3, 4, 9), (4, 3, 17), (6, 3, 5)])
@pytest.mark.parametrize("aug", [{}, dict(time_aug=True, end_time=2.5), dict(lead_lag=True),
                                 dict(time_aug=True, lead_lag=True, end_time=0.5)])
def test_forward_vs_independent_chen(d, deg, length, aug):
    rng = np.random.default_rng(7)
    x = rng.standard_normal((3, length, d))
    ref = M.signature_np(x, deg, **aug)
    for horner in (True, False):
        got = sigref.signature(x, deg, horner=horner, **aug)
        np.testing.assert_allclose(got, ref, rtol=1e-10, atol=1e-11)


def _tensor_mul(a, b, d, deg):
    """Chen product of two signatures given as flat arrays without scalar term."""
    sl = M.level_slices(d, deg)
    out = np.zeros_like(a)
    for t in range(1, deg + 1):
        acc = a[sl[t - 1]] + b[sl[t - 1]]
        for k in range(1, t):
            acc = acc + np.multiply.outer(a[sl[k - 1]], b[sl[t - k - 1]]).ravel()
        out[sl[t - 1]] = acc
    return out


def test_chen_time_reversal_reparam_shuffle():
    rng = np.random.default_rng(11)
    d, deg = 3, 4
    x = rng.standard_normal((9, d))
    full = sigref.signature(x, deg)
    # Chen: sig(x[:m+1]) (x) sig(x[m:]) == sig(x)
    m = 4
    np.testing.assert_allclose(_tensor_mul(sigref.signature(x[:m + 1], deg), sigref.signature(x[m:], deg), d, deg),
                               full, rtol=1e-11, atol=1e-12)
    # time reversal: sig(reversed) (x) sig(x) == 1
    rev = sigref.signature(x[::-1].copy(), deg)
    np.testing.assert_allclose(_tensor_mul(rev, full, d, deg), 0.0, atol=1e-10)
    # inserting collinear points changes nothing
    mid = 0.5 * (x[:-1] + x[1:])
    fine = np.empty((2 * len(x) - 1, d))
    fine[0::2], fine[1::2] = x, mid
    np.testing.assert_allclose(sigref.signature(fine, deg), full, rtol=1e-11, atol=1e-12)
    # shuffle identity at level 2: S^i S^j = S^{ij} + S^{ji}
    l1, l2 = full[:d], full[d:d + d * d].reshape(d, d)
    np.testing.assert_allclose(np.outer(l1, l1), l2 + l2.T, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("d,deg,length", [(2, 4, 6), (3, 3, 5), (2, 5, 4), (5, 2, 7), (1, 4, 5), (3, 1, 6)])
@pytest.mark.parametrize("aug", [{}, dict(time_aug=True, end_time=1.7), dict(lead_lag=True),
                                 dict(time_aug=True, lead_lag=True, end_time=3.0)])
def test_backward_vs_autograd(d, deg, length, aug):
    rng = np.random.default_rng(5 + d + deg)
    x = rng.standard_normal((2, length, d))
    sig = sigref.signature(x, deg, **aug)
    g = rng.standard_normal(sig.shape)
    ref = M.backprop_np(x, g, deg, **aug)
    for n_jobs in (1, -1):
        got = sigref.sig_backprop(x, sig, g, deg, n_jobs=n_jobs, **aug)
        np.testing.assert_allclose(got, ref, rtol=1e-9, atol=1e-10)
    got32 = sigref.sig_backprop(x.astype(np.float32), sig.astype(np.float32), g.astype(np.float32), deg, **aug)
    np.testing.assert_allclose(got32, ref, rtol=2e-3, atol=2e-3 * np.abs(ref).max())


def test_backward_finite_differences():
    rng = np.random.default_rng(3)
    d, deg = 3, 4
    x = rng.standard_normal((1, 6, d))
    sig = sigref.signature(x, deg)
    g = rng.standard_normal(sig.shape)
    grad = sigref.sig_backprop(x, sig, g, deg)
    direction = rng.standard_normal(x.shape)
    eps = 1e-5
    f = lambda y: float((sigref.signature(y, deg) * g).sum())
    fd = (f(x + eps * direction) - f(x - eps * direction)) / (2 * eps)
    assert abs(fd - float((grad * direction).sum())) <= 1e-7 * max(1.0, abs(fd))


def test_endpoint_only_gradients():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 7, 4))
    g = rng.standard_normal((2, 4))
    grad = sigref.sig_backprop(x, sigref.signature(x, 1), g, 1)
    np.testing.assert_array_equal(grad[:, 1:-1], 0.0)
    np.testing.assert_allclose(grad[:, -1], g)
    np.testing.assert_allclose(grad[:, 0], -g)


def test_trivial_and_error_cases():
    x = np.zeros((2, 1, 3))
    np.testing.assert_array_equal(sigref.signature(x, 2, scalar_term=True), [[1.] + [0.] * 12] * 2)
    np.testing.assert_array_equal(sigref.signature(x, 2), np.zeros((2, 12)))
    y = np.random.default_rng(0).standard_normal((2, 4, 3))
    np.testing.assert_array_equal(sigref.signature(y, 0, scalar_term=True), [[1.], [1.]])
    assert sigref.signature(y, 0).shape == (2, 0)
    np.testing.assert_array_equal(sigref.signature(y, 3, scalar_term=True)[:, 1:], sigref.signature(y, 3))
    np.testing.assert_array_equal(sigref.sig_backprop(x, np.zeros((2, 12)), np.ones((2, 12)), 2), 0.0)
    with pytest.raises(RuntimeError):
        sigref.signature(y, 2, n_jobs=0)


@pytest.mark.parametrize("batch", [1, 7, 8, 9, 16, 17])
def test_batch_chunking(batch):
    rng = np.random.default_rng(batch)
    x = rng.standard_normal((batch, 6, 3))
    a = sigref.signature(x, 3, n_jobs=1)
    b = sigref.signature(x, 3, n_jobs=-1)
    c = sigref.signature(x, 3, n_jobs=3)
    np.testing.assert_array_equal(a, b)
    np.testing.assert_array_equal(a, c)
