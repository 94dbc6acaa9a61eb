"""Pins the oracle's sig_combine / transform_path functions and their backward passes.

Evidence that does not come from the oracle: the reference's hand-computed vectors (tests/_ops_kats.py), its golden
float32 gradients of sig_combine (tests/golden/reference_fixture.npz, keys sig_comb_bp_*), Chen's identity against the
already pinned signature, an independent torch Chen product with autograd, and the textbook lead-lag / time
augmentation written with repeat / linspace.  linear_sig / sig_join (the reference holds no vectors for them): the
signature of the two-point path and of the path with one more point (the already pinned signature), the reference's
own statement sig_join == sig_combine(sig, linear_sig) (pysiglib/sig_join.py docstring), z^k/k! for one channel, and
autograd through the independent Chen product and segment exponential.
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


@pytest.mark.parametrize("d,deg", [(2, 6), (3, 4), (5, 3), (1, 7), (4, 1), (3, 0)])
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-13), (np.float32, 1e-5)])
def test_linear_sig_is_signature_of_a_segment(d, deg, dtype, tol):
    rng = np.random.default_rng(2 * d + deg)
    z = rng.standard_normal((4, d)).astype(dtype)
    got = sigref.linear_sig(z, d, deg, scalar_term=True)
    assert got.dtype == dtype and np.all(got[:, 0] == 1)
    np.testing.assert_array_equal(got[:, 1:], sigref.linear_sig(z, d, deg))
    if deg == 0:
        assert got.shape == (4, 1)
        return
    x = np.zeros((4, 2, d), dtype=dtype)
    x[:, 0] = rng.standard_normal((4, d)).astype(dtype)
    x[:, 1] = x[:, 0] + z
    z_eff = (x[:, 1] - x[:, 0]).astype(dtype)
    np.testing.assert_allclose(sigref.linear_sig(z_eff, d, deg), sigref.signature(x, deg), rtol=tol, atol=tol)
    # independent statement: z^(x)k / k!
    want = torch.cat(M._segment_exp(torch.tensor(z.astype(np.float64)), deg), dim=1).numpy()
    np.testing.assert_allclose(got[:, 1:], want, rtol=10 * tol, atol=10 * tol)
    if d == 1:
        fact = np.cumprod(np.arange(1, deg + 1, dtype=np.float64))
        np.testing.assert_allclose(got[:, 1:], z.astype(np.float64) ** np.arange(1, deg + 1) / fact, rtol=10 * tol, atol=tol)


@pytest.mark.parametrize("d,deg", [(2, 5), (3, 4), (5, 2), (1, 5), (4, 1)])
@pytest.mark.parametrize("prepend", [False, True])
def test_sig_join_extends_the_path(d, deg, prepend):
    rng = np.random.default_rng(d + 10 * deg)
    x = rng.uniform(size=(5, 9, d))
    z = rng.standard_normal((5, d))
    s = sigref.signature(x, deg)
    longer = np.concatenate([x[:, :1] - z[:, None], x], axis=1) if prepend else np.concatenate([x, x[:, -1:] + z[:, None]], axis=1)
    got = sigref.sig_join(s, z, d, deg, prepend=prepend)
    assert np.max(M.level_rel_err(got, sigref.signature(longer, deg), d, deg)) < 1e-11
    # the reference's own statement of the operator
    e = sigref.linear_sig(z, d, deg)
    want = sigref.sig_combine(e, s, d, deg) if prepend else sigref.sig_combine(s, e, d, deg)
    np.testing.assert_allclose(got, want, rtol=1e-13, atol=1e-13)
    # scalar-term layout and float32
    one = np.ones((5, 1))
    got1 = sigref.sig_join(np.hstack([one, s]), z, d, deg, prepend=prepend)
    assert np.all(got1[:, 0] == 1)
    np.testing.assert_array_equal(got1[:, 1:], got)
    gotf = sigref.sig_join(s.astype(np.float32), z.astype(np.float32), d, deg, prepend=prepend)
    assert gotf.dtype == np.float32
    np.testing.assert_allclose(gotf, got, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("d,deg", [(2, 5), (3, 4), (5, 2), (1, 5), (4, 1)])
@pytest.mark.parametrize("prepend", [False, True])
def test_sig_join_backprop_vs_autograd(d, deg, prepend):
    rng = np.random.default_rng(3 * d + deg)
    n = sigref.sig_length(d, deg) - 1
    a, g = rng.standard_normal((4, n)), rng.standard_normal((4, n))
    z = rng.standard_normal((4, d))
    ta, tz = torch.tensor(a, requires_grad=True), torch.tensor(z, requires_grad=True)
    e = M._segment_exp(tz, deg)
    out = M._chen(e, _levels(ta, d, deg), deg) if prepend else M._chen(_levels(ta, d, deg), e, deg)
    torch.cat(out, dim=1).backward(torch.tensor(g))
    ds, dz = sigref.sig_join_backprop(g, a, z, d, deg, prepend=prepend)
    np.testing.assert_allclose(ds, ta.grad.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dz, tz.grad.numpy(), rtol=1e-12, atol=1e-12)
    # scalar-term layout: same numbers, zero in the scalar slot
    one, zero = np.ones((4, 1)), np.zeros((4, 1))
    ds1, dz1 = sigref.sig_join_backprop(np.hstack([zero + 3.0, g]), np.hstack([one, a]), z, d, deg, prepend=prepend)
    assert np.all(ds1[:, 0] == 0)
    np.testing.assert_allclose(ds1[:, 1:], ds, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(dz1, dz, rtol=1e-13, atol=1e-13)
    dsf, dzf = sigref.sig_join_backprop(g.astype(np.float32), a.astype(np.float32), z.astype(np.float32), d, deg, prepend=prepend)
    np.testing.assert_allclose(dsf, ds, rtol=5e-4, atol=5e-4)
    np.testing.assert_allclose(dzf, dz, rtol=5e-4, atol=5e-4)


def test_sig_join_backprop_finite_differences():
    rng = np.random.default_rng(8)
    d, deg = 3, 4
    x = rng.uniform(size=(2, 6, d))
    s, z = sigref.signature(x, deg), rng.standard_normal((2, d))
    g = rng.standard_normal(s.shape)
    _, dz = sigref.sig_join_backprop(g, s, z, d, deg)
    h = 1e-6
    for j in range(d):
        zp, zm = z.copy(), z.copy()
        zp[:, j] += h
        zm[:, j] -= h
        num = ((sigref.sig_join(s, zp, d, deg) - sigref.sig_join(s, zm, d, deg)) * g).sum(axis=1) / (2 * h)
        np.testing.assert_allclose(dz[:, j], num, rtol=1e-6, atol=1e-7)


# ---------------------------------------------------------------------------
# sig_coef / sig_coef_backprop: pinned by the (already pinned) signature and its backward pass, which is also how the
# reference tests them (tests/test_sig_coef.py:46-55, tests/test_sig_coef_backprop.py), by the reference's trivial
# cases (tests/test_sig_coef.py:58-80) and by autograd through the independent Chen product.
# ---------------------------------------------------------------------------
def _widx(word, d):
    idx = 0
    for letter in word:
        idx = idx * d + letter + 1
    return idx - 1


def _all_words(d, degree):
    import itertools
    return [w for k in range(1, degree + 1) for w in itertools.product(range(d), repeat=k)]


COEF_AUGS = [{}, dict(time_aug=True, end_time=1.5), dict(lead_lag=True), dict(time_aug=True, lead_lag=True)]


def test_sig_coef_trivial_cases():
    x = np.array([[0., 0.], [1., 1.]])
    np.testing.assert_array_equal(sigref.sig_coef(x, [(0,), (1,)]), [1., 1.])
    np.testing.assert_array_equal(sigref.sig_coef(x[None], [(0,), (1,)]), [[1., 1.]])
    np.testing.assert_array_equal(sigref.sig_coef(x[:1], [(0,), (1,)]), [0., 0.])
    np.testing.assert_array_equal(sigref.sig_coef(x, [(), (0, 1)]), [1., 0.5])
    np.testing.assert_array_equal(sigref.sig_coef(x, [(), (0, 1)], prefixes=True), [1., 1., 0.5])


@pytest.mark.parametrize("aug", COEF_AUGS)
@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-12), (np.float32, 1e-4)])
def test_sig_coef_equals_signature_entries(aug, dtype, tol):
    rng = np.random.default_rng(21)
    d, deg = 2, 4
    x = rng.uniform(size=(3, 15, d)).astype(dtype)
    da = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    s = sigref.signature(x, deg, **aug)
    every = _all_words(da, 3)
    got = sigref.sig_coef(x, every, **aug)
    assert got.dtype == dtype
    np.testing.assert_allclose(got, s[:, :len(every)], rtol=tol, atol=tol)
    words = [(da - 1,), (0, da - 1), (1, 0, 1, da - 1), (da - 1, da - 1, 0), ()]
    got = sigref.sig_coef(x, words, **aug)
    want = np.stack([s[:, _widx(w, da)] if w else np.ones(3) for w in words], axis=1)
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol)
    pre = [w[:i] for w in words for i in range(1, len(w) + 1)] 
    gotp = sigref.sig_coef(x, words, prefixes=True, **aug)
    wantp = np.concatenate([np.stack([s[:, _widx(w[:i], da)] for i in range(1, len(w) + 1)], axis=1) if w else np.ones((3, 1))
                            for w in words], axis=1)
    assert gotp.shape == (3, len(pre) + 1)
    np.testing.assert_allclose(gotp, wantp, rtol=tol, atol=tol)


def test_sig_coef_long_word_closed_form():
    # one channel: the coefficient of the word (0,)*k is (x_end - x_0)^k / k!
    rng = np.random.default_rng(2)
    x = np.cumsum(rng.uniform(0.1, 0.3, size=(2, 9, 1)), axis=1)
    k = 24
    got = sigref.sig_coef(x, [(0,) * k], prefixes=True)
    inc = x[:, -1, 0] - x[:, 0, 0]
    fact = np.cumprod(np.arange(1, k + 1, dtype=np.float64))
    np.testing.assert_allclose(got, inc[:, None] ** np.arange(1, k + 1) / fact, rtol=1e-12, atol=0)


@pytest.mark.parametrize("aug", COEF_AUGS)
def test_sig_coef_backprop_equals_signature_backprop(aug):
    rng = np.random.default_rng(33)
    d, deg = 2, 4
    x = rng.uniform(size=(3, 8, d))
    da = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    words = [(da - 1,), (0, da - 1), (1, 0, 1, da - 1), (), (da - 1, da - 1, 0), (0, 0)]
    cp = sigref.sig_coef(x, words, prefixes=True, **aug)
    g = rng.standard_normal(cp.shape)
    s = sigref.signature(x, deg, **aug)
    G = np.zeros_like(s)
    col = 0
    for w in words:
        if not w:
            col += 1
            continue
        for i in range(1, len(w) + 1):
            G[:, _widx(w[:i], da)] += g[:, col]
            col += 1
    want = sigref.sig_backprop(x, s, G, deg, **aug)
    got = sigref.sig_coef_backprop(x, words, cp, g, **aug)
    np.testing.assert_allclose(got, want, rtol=1e-11, atol=1e-12)
    gotf = sigref.sig_coef_backprop(x.astype(np.float32), words, cp.astype(np.float32), g.astype(np.float32), **aug)
    assert gotf.dtype == np.float32
    np.testing.assert_allclose(gotf, want, rtol=2e-4, atol=2e-4)


def test_sig_coef_backprop_vs_autograd():
    rng = np.random.default_rng(34)
    d, deg = 3, 3
    words = [(2, 0, 1), (1, 1), (0,)]
    x = torch.tensor(rng.uniform(size=(2, 6, d)), requires_grad=True)
    s = M.signature(M.augment(x, time_aug=True, end_time=0.7), deg)
    cols = [_widx(w[:i], d + 1) for w in words for i in range(1, len(w) + 1)]
    g = rng.standard_normal((2, len(cols)))
    (s[:, cols] * torch.tensor(g)).sum().backward()
    xn = x.detach().numpy()
    cp = sigref.sig_coef(xn, words, prefixes=True, time_aug=True, end_time=0.7)
    np.testing.assert_allclose(cp, s[:, cols].detach().numpy(), rtol=1e-12, atol=1e-13)
    got = sigref.sig_coef_backprop(xn, words, cp, g, time_aug=True, end_time=0.7)
    np.testing.assert_allclose(got, x.grad.numpy(), rtol=1e-11, atol=1e-12)


# ---------------------------------------------------------------------------
# sig_to_log_sig (method 0) and its backward pass: the reference's golden vectors for the expanded log signature
# (tests/test_log_sig.py:101-144, tests/test_log_sig_backprop.py:49-100), the power series of log(1 + x) written with
# the independent Chen product, autograd through it, and log(exp(z)) = z.
# ---------------------------------------------------------------------------
def _log_series(levels, degree):
    """log(1 + x) = sum_n (-1)^(n+1) x^n / n with x given as level tensors (scalar part 0)."""
    B = levels[0].shape[0]

    def mul(a, b):      # product of two elements with zero scalar part
        out = []
        for t in range(1, degree + 1):
            acc = torch.zeros_like(levels[t - 1])
            for k in range(1, t):
                acc = acc + (a[k - 1].unsqueeze(2) * b[t - k - 1].unsqueeze(1)).reshape(B, -1)
            out.append(acc)
        return out

    power, total = levels, [l.clone() for l in levels]
    for n in range(2, degree + 1):
        power = mul(power, levels)
        total = [t + ((-1) ** (n + 1)) * p / n for t, p in zip(total, power)]
    return total


@pytest.mark.parametrize("deg", range(1, 6))
def test_log_sig_golden(fixtures, deg):
    x = fixtures["path"]
    for key, kw, d in (("logsig_exp", {}, 3), ("logsig_exp_ta", dict(time_aug=True), 4)):
        s = sigref.signature(x, deg, **kw)
        np.testing.assert_allclose(sigref.sig_to_log_sig(s, d, deg), fixtures["%s__d%d" % (key, deg)], rtol=0, atol=1e-10)
        one = np.hstack([np.ones((len(s), 1)), s])
        got1 = sigref.sig_to_log_sig(one, d, deg)
        assert np.all(got1[:, 0] == 0)
        np.testing.assert_array_equal(got1[:, 1:], sigref.sig_to_log_sig(s, d, deg))
    if deg <= 4:
        s = sigref.signature(x[:2], deg, lead_lag=True)
        np.testing.assert_allclose(sigref.sig_to_log_sig(s, 6, deg), fixtures["logsig_exp_ll__d%d" % deg], rtol=0, atol=1e-10)
    sf = sigref.signature(x.astype(np.float32), deg)
    gotf = sigref.sig_to_log_sig(sf, 3, deg)
    assert gotf.dtype == np.float32
    np.testing.assert_allclose(gotf, fixtures["logsig_exp__d%d" % deg], rtol=0, atol=1e-4)


@pytest.mark.parametrize("deg", range(1, 6))
def test_log_sig_backprop_golden(fixtures, deg):
    # the reference checks the path gradient through log_sig(method=0): tensor-log adjoint, then the pinned sig_backprop
    x = fixtures["path"]
    for key, kw, d in (("logsig_bp_exp", {}, 3), ("logsig_bp_exp_ta", dict(time_aug=True), 4)):
        s = sigref.signature(x, deg, **kw)
        ds = sigref.sig_to_log_sig_backprop(s, fixtures["%s_derivs__d%d" % (key, deg)], d, deg)
        got = sigref.sig_backprop(x, s, ds, deg, **kw)
        np.testing.assert_allclose(got, fixtures["%s_expected__d%d" % (key, deg)], rtol=0, atol=1e-5)


# ---- compressed log signatures: Lyndon words (method 1) and Lyndon basis (method 2) -----------------------------

def _witt(d, n):
    """Number of Lyndon words of length n over d letters (necklace polynomial)."""
    def mobius(k):
        res, p = 1, 2
        while p * p <= k:
            if k % p == 0:
                k //= p
                if k % p == 0:
                    return 0
                res = -res
            p += 1
        return -res if k > 1 else res
    return sum(mobius(n // x) * d ** x for x in range(1, n + 1) if n % x == 0) // n


@pytest.mark.parametrize("d,deg", [(2, 7), (3, 5), (5, 4), (1, 4), (7, 3)])
def test_lyndon_words(d, deg):
    from oracle import lyndon
    words = lyndon.lyndon_words(d, deg)
    # counts by the necklace polynomial; every word strictly smaller than its proper suffixes; sorted inside a length
    for n in range(1, deg + 1):
        level = [w for w in words if len(w) == n]
        assert len(level) == _witt(d, n)
        assert level == sorted(level)
        for w in level:
            assert all(w < w[i:] for i in range(1, n))
    assert [len(w) for w in words] == sorted(len(w) for w in words)
    # brute force: nothing is missing
    if d ** deg <= 3000:
        import itertools
        brute = [w for n in range(1, deg + 1) for w in itertools.product(range(d), repeat=n)
                 if all(w < w[i:] for i in range(1, n))]
        assert set(brute) == set(words)
    # the projection is unit lower triangular and couples only words made of the same letters
    m = lyndon.projection_matrix(d, deg)
    assert np.all(np.diag(m) == 1) and np.all(np.triu(m, 1) == 0)
    for i, j in zip(*np.nonzero(m)):
        assert sorted(words[i]) == sorted(words[j])


@pytest.mark.parametrize("deg", range(1, 6))
def test_log_sig_lyndon_golden(fixtures, deg):
    # signatory's "words" mode and iisignature's "s" (Lyndon basis) coordinates, held by the reference's fixture
    x = fixtures["path"]
    s = sigref.signature(x, deg)
    np.testing.assert_allclose(sigref.sig_to_log_sig(s, 3, deg, method=1), fixtures["logsig_words__d%d" % deg], rtol=0, atol=1e-12)
    np.testing.assert_allclose(sigref.sig_to_log_sig(s, 3, deg, method=2), fixtures["logsig_basis__d%d" % deg], rtol=0, atol=1e-12)
    one = np.hstack([np.ones((len(s), 1)), s])
    for method in (1, 2):
        np.testing.assert_array_equal(sigref.sig_to_log_sig(one, 3, deg, method=method), sigref.sig_to_log_sig(s, 3, deg, method=method))
    # path gradients through the compressed coordinates
    for name, method, tol in (("words", 1, 1e-10), ("basis", 2, 1e-5)):
        ds = sigref.sig_to_log_sig_backprop(s, fixtures["logsig_bp_%s_derivs__d%d" % (name, deg)], 3, deg, method=method)
        got = sigref.sig_backprop(x, s, ds, deg)
        np.testing.assert_allclose(got, fixtures["logsig_bp_%s_expected__d%d" % (name, deg)], rtol=0, atol=tol)


@pytest.mark.parametrize("d,deg", [(2, 6), (3, 4), (4, 3)])
def test_log_sig_lyndon_basis_reconstructs(d, deg):
    """The log signature of a path is a Lie element: expanding its Lyndon-basis coordinates through the brackets
    must give back the whole expanded log signature, not only its Lyndon-word coefficients; and the backward passes
    of both methods are the transposes of the forward maps."""
    from oracle import lyndon
    rng = np.random.default_rng(d + deg)
    x = np.cumsum(rng.standard_normal((3, 12, d)), axis=1) * 0.3
    s = sigref.signature(x, deg)
    expanded = sigref.sig_to_log_sig(s, d, deg)
    beta = sigref.sig_to_log_sig(s, d, deg, method=2)
    words = lyndon.lyndon_words(d, deg)
    poly = lyndon._bracket_polynomials(words)
    rebuilt = np.zeros_like(expanded)
    for j, w in enumerate(words):
        for word, c in poly[w].items():
            rebuilt[:, lyndon.word_index(word, d)] += c * beta[:, j]
    np.testing.assert_allclose(rebuilt, expanded, rtol=0, atol=1e-12)
    n = expanded.shape[1]
    for method in (1, 2):
        m = len(words)
        fwd = np.stack([lyndon.compress(e, d, deg, method) for e in np.eye(n)], axis=1)          # (m, n) matrix
        bwd = np.stack([lyndon.compress_backprop(e, d, deg, method) for e in np.eye(m)], axis=0)  # (m, n) as well
        np.testing.assert_allclose(bwd, fwd, rtol=0, atol=1e-13)


@pytest.mark.parametrize("d,deg", [(2, 6), (3, 4), (5, 3), (1, 5), (4, 1), (3, 2)])
def test_log_sig_vs_power_series_and_autograd(d, deg):
    rng = np.random.default_rng(d * 7 + deg)
    n = sigref.sig_length(d, deg) - 1
    a = rng.standard_normal((3, n)) * 0.5           # arbitrary tensors, not group-like
    g = rng.standard_normal((3, n))
    ta = torch.tensor(a, requires_grad=True)
    want = torch.cat(_log_series(_levels(ta, d, deg), deg), dim=1)
    np.testing.assert_allclose(sigref.sig_to_log_sig(a, d, deg), want.detach().numpy(), rtol=1e-12, atol=1e-12)
    want.backward(torch.tensor(g))
    got = sigref.sig_to_log_sig_backprop(a, g, d, deg)
    np.testing.assert_allclose(got, ta.grad.numpy(), rtol=1e-11, atol=1e-11)
    one, zero = np.ones((3, 1)), np.zeros((3, 1))
    got1 = sigref.sig_to_log_sig_backprop(np.hstack([one, a]), np.hstack([zero + 5.0, g]), d, deg)
    assert np.all(got1[:, 0] == 0)
    np.testing.assert_allclose(got1[:, 1:], got, rtol=1e-13, atol=1e-13)
    gotf = sigref.sig_to_log_sig_backprop(a.astype(np.float32), g.astype(np.float32), d, deg)
    np.testing.assert_allclose(gotf, got, rtol=1e-3, atol=1e-3)


def test_log_of_segment_exponential_is_the_increment():
    rng = np.random.default_rng(4)
    d, deg = 3, 5
    z = rng.standard_normal((4, d))
    lg = sigref.sig_to_log_sig(sigref.linear_sig(z, d, deg), d, deg)
    np.testing.assert_allclose(lg[:, :d], z, rtol=0, atol=1e-14)
    np.testing.assert_allclose(lg[:, d:], 0, rtol=0, atol=1e-13)
