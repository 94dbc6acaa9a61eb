"""Parity of the HIP path (through the C ABI) with the CPU oracle and the golden vectors.

Tolerances: float64 1e-10, float32 1e-4, relative to the per-level (forward) or per-path (backward) max norm,
as stated for this path; the golden-vector tests use the reference's absolute tolerances
(tests/conftest.py:34-50 of the reference: 1e-10 / 1e-4; backward fixtures are float32, 1e-5).
"""
import warnings

import numpy as np
import pytest
import torch

from pysiglib_amd import workloads as C
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


def dev(a):
    return torch.tensor(np.ascontiguousarray(a), device=DEV)


def bwd_rel_err(got, ref):
    got = got.reshape(ref.shape[0], -1).astype(np.float64)
    ref2 = ref.reshape(ref.shape[0], -1).astype(np.float64)
    den = np.maximum(np.abs(ref2).max(axis=1), np.finfo(np.float64).tiny)
    return float((np.abs(got - ref2).max(axis=1) / den).max())


AUGS = {
    "sig": ({}, "path"),
    "sig_ta": (dict(time_aug=True), "path"),
    "sig_ll": (dict(lead_lag=True), "path_dim2"),
    "sig_ta_ll": (dict(time_aug=True, lead_lag=True), "path_dim2"),
}


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("key", list(AUGS))
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_forward_golden(P, fixtures, deg, key, dtype):
    kw, pkey = AUGS[key]
    expected = fixtures[f"{key}__d{deg}"]
    x = fixtures[pkey].astype(dtype)
    got = P.sig(dev(x), deg, **kw)
    assert got.device.type == "cuda"
    np.testing.assert_allclose(got.cpu().numpy(), expected, rtol=0, atol=TOL[dtype])
    single = P.sig(dev(x[0]), deg, horner=False, **kw)          # single path, other value of the horner flag
    np.testing.assert_allclose(single.cpu().numpy(), expected[0], rtol=0, atol=TOL[dtype])


@pytest.mark.parametrize("deg", range(1, 6))
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_backward_golden(P, fixtures, deg, dtype):
    x = dev(fixtures["path"].astype(dtype))
    g = dev(fixtures[f"sig_bp_derivs__d{deg}"].astype(dtype))     # one column wider: carries the scalar slot
    expected = fixtures[f"sig_bp_expected__d{deg}"]
    s = P.sig(x, deg)
    got = P.sig_backprop(x.clone(), s.clone(), g.clone(), deg)
    np.testing.assert_allclose(got.cpu().numpy(), expected, rtol=0, atol=1e-5 if dtype == np.float64 else 1e-4)


def test_kats(P, kats):
    for k in kats["forward"]:
        if k["length"] == 0:
            continue    # zero-length tensors cannot carry the shape through torch
        dt = np.dtype(k["dtype"]).type
        x = np.array(k["path"], dtype=dt).reshape(k["batch"], k["length"], k["dimension"])
        got = P.sig(dev(x), k["degree"], time_aug=k["time_aug"], lead_lag=k["lead_lag"], end_time=k["end_time"],
                    scalar_term=True).cpu().numpy()
        tol = 1e-12 if dt == np.float64 else 2e-5
        np.testing.assert_allclose(got.ravel(), np.array(k["expected"]), rtol=tol, atol=tol, err_msg=k["name"])
    for k in kats["backward"]:
        x = np.array(k["path"]).reshape(k["batch"], k["length"], k["dimension"])
        s = np.array(k["sig"]).reshape(k["batch"], -1)
        g = np.array(k["derivs"]).reshape(k["batch"], -1)
        got = P.sig_backprop(dev(x), dev(s), dev(g), k["degree"], time_aug=k["time_aug"], lead_lag=k["lead_lag"],
                             end_time=k["end_time"]).cpu().numpy()
        np.testing.assert_allclose(got.ravel(), np.array(k["expected"]), rtol=1e-12, atol=1e-12, err_msg=k["name"])


# (batch, length, dim, degree): specialised kernels, run-time-dimension kernel, batch tails, wide/packed geometries
GRID = [
    (1, 2, 2, 2), (3, 6, 2, 6), (7, 9, 3, 4), (9, 5, 4, 4), (17, 12, 3, 3), (70, 6, 2, 3), (2, 33, 5, 4),
    (3, 10, 6, 3), (2, 10, 7, 4), (2, 6, 20, 2), (1, 8, 37, 3), (4, 5, 2, 13), (2, 12, 3, 9), (130, 4, 3, 2),
    (2, 40, 10, 5), (2, 40, 5, 7), (1, 25, 3, 12), (2, 15, 17, 4), (3, 7, 16, 3), (2, 9, 9, 4), (5, 6, 2, 16),
]


@pytest.mark.parametrize("shape", GRID)
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_grid_vs_oracle(P, oracle, shape, dtype, scalar_term):
    b, length, d, deg = shape
    rng = np.random.default_rng(hash(shape) % (2 ** 31))
    x = (rng.standard_normal((b, length, d)) * (0.5 if deg > 6 else 1.0)).astype(dtype)
    ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1)
    got = P.sig(dev(x), deg, scalar_term=scalar_term).cpu().numpy()
    off = 1 if scalar_term else 0
    if scalar_term:
        np.testing.assert_array_equal(got[:, 0], 1.0)
    assert level_rel_err(got[:, off:], ref[:, off:], d, deg) <= TOL[dtype]
    g = rng.standard_normal(ref.shape).astype(dtype)
    ref_b = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
    xt, st, gt = dev(x), dev(ref), dev(g)
    keep = (xt.clone(), st.clone(), gt.clone())
    got_b = P.sig_backprop(xt, st, gt, deg).cpu().numpy()
    assert bwd_rel_err(got_b, ref_b) <= TOL[dtype]
    for a, bb in zip((xt, st, gt), keep):       # inputs are left bit-identical
        assert torch.equal(a, bb)


@pytest.mark.parametrize("aug", [dict(time_aug=True, end_time=2.5), dict(lead_lag=True),
                                 dict(time_aug=True, lead_lag=True, end_time=0.5)])
@pytest.mark.parametrize("shape", [(3, 9, 2, 4), (2, 12, 3, 3), (5, 7, 1, 5), (2, 20, 8, 4), (2, 6, 4, 2), (3, 5, 3, 1)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_augmentations_vs_oracle(P, oracle, aug, shape, dtype):
    b, length, d, deg = shape
    rng = np.random.default_rng(17 + d + deg)
    x = (rng.standard_normal((b, length, d)) * 0.7).astype(dtype)
    d_aug = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    ref = oracle.signature(x, deg, n_jobs=-1, **aug)
    got = P.sig(dev(x), deg, **aug).cpu().numpy()
    assert level_rel_err(got, ref, d_aug, deg) <= TOL[dtype]
    g = rng.standard_normal(ref.shape).astype(dtype)
    ref_b = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, **aug)
    got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
    assert bwd_rel_err(got_b, ref_b) <= TOL[dtype]


def test_closed_forms(P):
    # straight line: level k = v^(x)k / k!   (tests/test_cuda_horner.py:100-112 of the reference)
    rng = np.random.default_rng(5)
    for d, deg in ((2, 12), (3, 8), (5, 5), (10, 4)):
        v = rng.standard_normal(d) * 0.8
        ts = np.linspace(0, 1, 9) ** 2
        got = P.sig(dev(ts[:, None] * v[None, :]), deg).cpu().numpy()
        lvl, off = np.array(1.0), 0
        for k in range(1, deg + 1):
            lvl = np.multiply.outer(lvl, v) / k
            np.testing.assert_allclose(got[off:off + d ** k], lvl.ravel(), rtol=1e-11, atol=1e-14)
            off += d ** k
    # d = 1: Delta^k / k!
    import math
    x = np.array([[0.3], [1.0], [-2.0], [0.7]])
    np.testing.assert_allclose(P.sig(dev(x), 6, scalar_term=True).cpu().numpy(),
                               [0.4 ** k / math.factorial(k) for k in range(7)], rtol=1e-13)
    # degree 1 / d = 1: only the endpoints receive gradient, interior exactly zero
    y = dev(rng.standard_normal((2, 7, 4)))
    g = dev(rng.standard_normal((2, 4)))
    grad = P.sig_backprop(y, P.sig(y, 1), g, 1)
    assert torch.equal(grad[:, 1:-1], torch.zeros_like(grad[:, 1:-1]))
    torch.testing.assert_close(grad[:, -1], g)
    torch.testing.assert_close(grad[:, 0], -g)


def test_trivial_cases(P):
    x = torch.zeros(2, 1, 3, dtype=torch.float64, device=DEV)
    assert torch.equal(P.sig(x, 2, scalar_term=True).cpu(), torch.tensor([[1.] + [0.] * 12] * 2, dtype=torch.float64))
    assert torch.equal(P.sig(x, 2).cpu(), torch.zeros(2, 12, dtype=torch.float64))
    y = torch.randn(2, 4, 3, dtype=torch.float64, device=DEV)
    assert torch.equal(P.sig(y, 0, scalar_term=True).cpu(), torch.ones(2, 1, dtype=torch.float64))
    assert P.sig(y, 0).shape == (2, 0)
    assert torch.equal(P.sig(y, 3, scalar_term=True)[:, 1:], P.sig(y, 3))
    assert torch.equal(P.sig_backprop(x, torch.zeros(2, 12, dtype=torch.float64, device=DEV),
                                      torch.ones(2, 12, dtype=torch.float64, device=DEV), 2).cpu(),
                       torch.zeros(2, 1, 3, dtype=torch.float64))
    assert P.sig(torch.zeros(0, 5, 3, dtype=torch.float64, device=DEV), 3).shape == (0, 39)
    two = torch.tensor([[0., 0.], [1., 1.]], device=DEV)
    torch.testing.assert_close(P.sig(two, 1).cpu(), torch.tensor([1., 1.]))


def test_batch_dims_views_and_warnings(P, oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 8, 4))
    ref = oracle.signature(x.reshape(6, 8, 4), 3).reshape(2, 3, -1)
    got = P.sig(dev(x), 3)
    assert got.shape == (2, 3, 84)
    np.testing.assert_allclose(got.cpu().numpy(), ref, rtol=1e-11, atol=1e-12)
    g = rng.standard_normal(ref.shape)
    ref_b = oracle.sig_backprop(x.reshape(6, 8, 4), ref.reshape(6, -1), g.reshape(6, -1), 3).reshape(x.shape)
    np.testing.assert_allclose(P.sig_backprop(dev(x), dev(ref), dev(g), 3).cpu().numpy(), ref_b, rtol=1e-10, atol=1e-11)
    # non-contiguous / expanded inputs are cloned (tests/test_signature.py:58-79 of the reference)
    base = torch.rand(5, 20, dtype=torch.float64, device=DEV)[:, :, None]
    view = base.expand(-1, -1, 6)
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        torch.testing.assert_close(P.sig(view, 3), P.sig(view.clone(), 3))
        strided = torch.randn(4, 30, 6, dtype=torch.float64, device=DEV)[..., ::2]
        torch.testing.assert_close(P.sig(strided, 4), P.sig(strided.contiguous(), 4))
    # overflow in the result warns (pysiglib/sig.py:299-310)
    with pytest.warns(RuntimeWarning):
        P.sig(torch.full((1, 3, 2), 1e200, dtype=torch.float64, device=DEV).cumsum(1), 3)


def test_point_fed_staging(P):
    """Staged forward sweeps of plain paths of at most 16 channels difference the points while staging them; the
    result must equal, bit for bit, the sweep fed by the increments kernel (same subtractions, same order), for
    lengths around the 16-step chunk, forced time segments and the last path of the batch (whose final chunk must
    not read past the end of the path buffer)."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_point_fed.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_point_fed.restype = None
    L.CUSIG.cusig_amd_force_staged.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_staged.restype = None
    rng = np.random.default_rng(4242)
    fed = 0
    try:
        L.CUSIG.cusig_amd_force_staged(1)
        for (d, n) in ((10, 5), (5, 7), (4, 8), (16, 4), (17, 4), (12, 4), (6, 6)):
            for length in (2, 3, 16, 17, 18, 33, 100):
                for segments in (0, 3):
                    for dtype in (torch.float64, torch.float32):
                        x = torch.as_tensor(rng.standard_normal((48, length, d)), dtype=dtype, device=DEV)
                        L.CUSIG.cusig_amd_force_segments(segments)
                        L.CUSIG.cusig_amd_set_point_fed(0)
                        ref = P.sig(x, n)
                        L.CUSIG.cusig_amd_set_point_fed(1)
                        L.CUSIG.cusig_amd_set_profiling(1)
                        out = P.sig(x, n)
                        name = L.CUSIG.cusig_amd_last_kernel_name().decode()
                        L.CUSIG.cusig_amd_set_profiling(0)
                        fed += name.endswith("_lds") and d <= 16
                        assert torch.equal(out, ref), (d, n, length, segments, dtype, name)
        # augmented paths keep the increments kernel: same answers either way
        x = torch.as_tensor(rng.standard_normal((3, 20, 4)), dtype=torch.float64, device=DEV)
        L.CUSIG.cusig_amd_set_point_fed(0)
        ref = P.sig(x, 4, time_aug=True, lead_lag=True)
        L.CUSIG.cusig_amd_set_point_fed(1)
        assert torch.equal(P.sig(x, 4, time_aug=True, lead_lag=True), ref)
    finally:
        L.CUSIG.cusig_amd_force_segments(0)
        L.CUSIG.cusig_amd_set_point_fed(1)
        L.CUSIG.cusig_amd_force_staged(-1)
    assert fed > 100     # the staged kernels did run


def test_point_fed_backward(P, oracle):
    """Staged backward sweeps of plain paths of at most 16 channels form the increments from the points as well, and
    their increment-gradient accumulators take turns (each call's last launch clears the other one): against the sweep
    fed by the increments kernel and against the oracle, for lengths around the 16-step chunk, shapes that change from
    call to call (growing and shrinking accumulators), both precisions, and the last path of the batch."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_point_fed.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_point_fed.restype = None
    L.CUSIG.cusig_amd_force_staged.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_staged.restype = None
    rng = np.random.default_rng(4343)
    fed = 0
    try:
        L.CUSIG.cusig_amd_force_staged(1)
        for (d, n) in ((10, 5), (5, 7), (4, 8), (16, 4), (17, 4), (12, 4), (6, 6)):
            for length, batch in ((2, 3), (3, 48), (16, 5), (17, 48), (18, 2), (33, 48), (100, 7), (40, 64)):
                for dtype in (np.float64, np.float32):
                    x = (rng.standard_normal((batch, length, d)) * 0.4).astype(dtype)
                    sig = P.sig(dev(x), n)
                    g = dev(rng.standard_normal(tuple(sig.shape)).astype(dtype))
                    L.CUSIG.cusig_amd_set_point_fed(0)
                    ref = P.sig_backprop(dev(x), sig, g, n).cpu().numpy()
                    L.CUSIG.cusig_amd_set_point_fed(1)
                    L.CUSIG.cusig_amd_set_profiling(1)
                    out = P.sig_backprop(dev(x), sig, g, n).cpu().numpy()
                    name = L.CUSIG.cusig_amd_last_kernel_name().decode()
                    L.CUSIG.cusig_amd_set_profiling(0)
                    fed += name.endswith("_lds") and d <= 16
                    # the same sums in another order of the atomic adds: rounding-level agreement
                    assert bwd_rel_err(out, ref) <= (1e-13 if dtype == np.float64 else 2e-5), (d, n, length, batch, dtype, name)
                    if length in (17, 40):
                        want = oracle.sig_backprop(x, sig.cpu().numpy(), g.cpu().numpy(), n, n_jobs=-1)
                        assert bwd_rel_err(out, want) <= TOL[dtype], (d, n, length, batch, dtype, name)
    finally:
        L.CUSIG.cusig_amd_set_point_fed(1)
        L.CUSIG.cusig_amd_force_staged(-1)
    assert fed > 40      # the staged kernels did run


def test_lead_lag_sparse_steps(P, oracle):
    """Staged forward sweeps of lead-lag paths leave out the multiply-adds by the channels a step cannot move (their
    increments are exactly zero): same bits as the dense sweep of the same pieces, for both time-augmentation settings,
    odd and even lengths, forced time segments (which must start on even steps), and against the oracle."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_lead_lag_sparse.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_lead_lag_sparse.restype = None
    L.CUSIG.cusig_amd_force_staged.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_staged.restype = None
    rng = np.random.default_rng(777)
    ran = 0
    try:
        L.CUSIG.cusig_amd_force_staged(1)
        for (d_raw, n) in ((8, 4), (2, 6), (3, 5), (5, 4), (4, 3), (10, 3), (2, 8)):
            for time_aug in (False, True):
                for length in (2, 3, 8, 9, 17, 40):
                    for segments in (0, 3):
                        for dtype in (torch.float64, torch.float32):
                            x = torch.as_tensor(rng.standard_normal((40, length, d_raw)).cumsum(1) * 0.3, dtype=dtype, device=DEV)
                            kw = dict(time_aug=time_aug, lead_lag=True)
                            L.CUSIG.cusig_amd_force_segments(segments)
                            L.CUSIG.cusig_amd_set_lead_lag_sparse(0)
                            ref = P.sig(x, n, **kw)
                            pieces = L.CUSIG.cusig_amd_last_segments()
                            L.CUSIG.cusig_amd_set_lead_lag_sparse(1)
                            L.CUSIG.cusig_amd_set_profiling(1)
                            out = P.sig(x, n, **kw)
                            name = L.CUSIG.cusig_amd_last_kernel_name().decode()
                            L.CUSIG.cusig_amd_set_profiling(0)
                            ran += name.endswith("_ll")
                            if pieces == 1 and L.CUSIG.cusig_amd_last_segments() == 1:
                                assert torch.equal(out, ref), (d_raw, n, time_aug, length, segments, dtype, name)
                            else:       # pieces of even length may be cut elsewhere: another order of additions
                                tol = 1e-12 if dtype == torch.float64 else 2e-5
                                scale = ref.abs().max().item()
                                assert (out - ref).abs().max().item() <= tol * max(scale, 1.0), (d_raw, n, time_aug, length, segments, dtype, name)
        x = rng.standard_normal((256, 21, 4)).cumsum(1) * 0.3
        for time_aug in (False, True):
            want = oracle.signature(x, 4, time_aug=time_aug, lead_lag=True)
            got = P.sig(dev(x), 4, time_aug=time_aug, lead_lag=True).cpu().numpy()
            assert level_rel_err(got, want, 8 + int(time_aug), 4) <= 1e-10
    finally:
        L.CUSIG.cusig_amd_force_segments(0)
        L.CUSIG.cusig_amd_set_lead_lag_sparse(1)
        L.CUSIG.cusig_amd_force_staged(-1)
        L.CUSIG.cusig_amd_set_profiling(0)
    assert ran > 100     # the lead-lag twins did run


def test_lead_lag_sparse_backward(P, oracle):
    """Staged backward sweeps of lead-lag paths leave out, per step, the multiply-adds of the channels that step cannot
    move (their increments are zero and their increment gradients are never read): same bits as the dense sweep when
    both run the path in one piece, within tolerance when forced time pieces are cut at different (even) steps, and
    parity with the oracle."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_bwd_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_bwd_segments.restype = None
    L.CUSIG.cusig_amd_set_lead_lag_sparse.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_lead_lag_sparse.restype = None
    L.CUSIG.cusig_amd_force_staged.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_staged.restype = None
    rng = np.random.default_rng(778)
    ran = 0
    ran_direct = 0
    try:
        # staged kernels, then the scalar-fed ones (which have a lead-lag form from 14 channels on in double precision
        # and from 32 on in single precision, where the mask acts on the subtree level below the lane's own letters)
        cases = [(1, d_raw, n, 40) for (d_raw, n) in ((8, 4), (2, 6), (3, 5), (5, 4), (4, 3), (10, 3), (2, 8), (15, 3))]
        cases += [(0, d_raw, n, b) for (d_raw, n, b) in ((7, 3, 64), (8, 4, 48), (10, 3, 70), (10, 4, 40), (12, 4, 24))]
        for (staged, d_raw, n, batch) in cases:
            L.CUSIG.cusig_amd_force_staged(staged)
            for time_aug in (False, True):
                for length in (2, 3, 8, 9, 17, 40):
                    for segments in (0, 3):
                        for dtype in (torch.float64, torch.float32):
                            x = torch.as_tensor(rng.standard_normal((batch, length, d_raw)).cumsum(1) * 0.3, dtype=dtype, device=DEV)
                            kw = dict(time_aug=time_aug, lead_lag=True)
                            sg = P.sig(x, n, **kw)
                            g = torch.as_tensor(rng.standard_normal(tuple(sg.shape)), dtype=dtype, device=DEV)
                            L.CUSIG.cusig_amd_force_bwd_segments(segments)
                            L.CUSIG.cusig_amd_set_lead_lag_sparse(0)
                            ref = P.sig_backprop(x, sg, g, n, **kw)
                            L.CUSIG.cusig_amd_set_lead_lag_sparse(1)
                            L.CUSIG.cusig_amd_set_profiling(1)
                            out = P.sig_backprop(x, sg, g, n, **kw)
                            name = L.CUSIG.cusig_amd_last_kernel_name().decode()
                            L.CUSIG.cusig_amd_set_profiling(0)
                            ran += name.endswith("_lds_ll")
                            ran_direct += name.endswith("_ll") and not name.endswith("_lds_ll")
                            case = (d_raw, n, time_aug, length, segments, dtype, name)
                            if segments == 0 and length < 32:     # one piece either way; pieces share atomics otherwise
                                tol = 1e-13 if dtype == torch.float64 else 2e-5     # float atomics land in any order
                            else:
                                tol = 1e-11 if dtype == torch.float64 else 1e-4
                            scale = ref.abs().max().item()
                            assert (out - ref).abs().max().item() <= tol * max(scale, 1.0), case
        L.CUSIG.cusig_amd_force_staged(-1)
        for (d_raw, n, length) in ((4, 4, 21), (3, 5, 12), (8, 3, 30), (8, 4, 14), (10, 3, 11)):
            x = rng.standard_normal((64 if d_raw < 8 or n < 4 else 6, length, d_raw)).cumsum(1) * 0.3
            for time_aug in (False, True):
                aug = dict(time_aug=time_aug, lead_lag=True)
                ref = oracle.signature(x, n, **aug)
                g = rng.standard_normal(ref.shape)
                want = oracle.sig_backprop(x, ref, g, n, n_jobs=-1, **aug)
                for segments in (0, 4):
                    L.CUSIG.cusig_amd_force_bwd_segments(segments)
                    got = P.sig_backprop(dev(x), dev(ref), dev(g), n, **aug).cpu().numpy()
                    assert bwd_rel_err(got, want) <= 1e-10, (d_raw, n, length, time_aug, segments)
    finally:
        L.CUSIG.cusig_amd_force_bwd_segments(0)
        L.CUSIG.cusig_amd_set_lead_lag_sparse(1)
        L.CUSIG.cusig_amd_force_staged(-1)
        L.CUSIG.cusig_amd_set_profiling(0)
    assert ran > 100 and ran_direct > 50     # the lead-lag twins of both kinds did run


def test_overflow_report(P):
    """The kernels that store the signature flag NaN / Inf themselves (the reference scans the result,
    pysiglib/sig.py:299-310): the report must agree with a scan on every forward route."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_stream_ordered.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_stream_ordered.restype = None
    rng = np.random.default_rng(77)
    shapes = [(3, 20, 3, 4), (2, 40, 10, 5), (70, 9, 2, 3), (2, 12, 20, 3), (2, 12, 40, 2),     # packed, wide, many per wave, generic
              (4, 9, 1, 5), (4, 9, 6, 1), (3, 1, 4, 3)]                                       # dimension one, degree one, single point
    for segments in (0, 3):
        try:
            L.CUSIG.cusig_amd_force_segments(segments)
            for shape in shapes:
                for dtype in (torch.float64, torch.float32):
                    big = 1e200 if dtype == torch.float64 else 1e30
                    for kind in ("finite", "overflow", "nan"):
                        x = torch.as_tensor(rng.standard_normal(shape[:3]), dtype=dtype, device=DEV)
                        if kind == "overflow":
                            x[shape[0] - 1] *= big        # only the last path
                        elif kind == "nan":
                            x[0, shape[1] // 2, 0] = float("nan")
                        with warnings.catch_warnings(record=True) as caught:
                            warnings.simplefilter("always")
                            out = P.sig(x, shape[3], scalar_term=bool(shape[0] % 2))
                        warned = any(issubclass(w.category, RuntimeWarning) for w in caught)
                        assert L.CUSIG.cusig_amd_last_sig_nonfinite() in (0, 1)
                        assert warned == (not bool(torch.isfinite(out).all())), (shape, dtype, kind, segments)
        finally:
            L.CUSIG.cusig_amd_force_segments(0)
    # stream-ordered calls cannot know at return: no report, the wrapper scans
    try:
        L.CUSIG.cusig_amd_set_stream_ordered(1)
        with pytest.warns(RuntimeWarning):
            P.sig(torch.full((1, 3, 2), 1e200, dtype=torch.float64, device=DEV).cumsum(1), 3)
        assert L.CUSIG.cusig_amd_last_sig_nonfinite() == -1
    finally:
        L.CUSIG.cusig_amd_set_stream_ordered(0)


def test_error_codes_through_the_abi(P):
    import ctypes
    from pysiglib_amd import _loader as L
    f = L.CUSIG_SIGNATURE["float64"]
    x = torch.zeros(8, dtype=torch.float64, device=DEV)
    p = ctypes.cast(x.data_ptr(), ctypes.POINTER(ctypes.c_double))
    assert f(p, p, 1, 0, 2, 2, False, False, 1.0, True, True, None, 0, 0, 0) == 2          # dimension 0
    assert "dimension 0" in L.last_error_message()
    assert f(p, p, 1, 2, 2, 2, False, False, 1.0, True, True, None, 4, 0, 0) == 2          # null correction, len != 0
    assert f(p, p, 1, 2, 2, 2, False, True, 1.0, True, True, p, 4, 0, 0) == 2              # correction with lead-lag
    assert f(p, p, 1, 2, 2, 2, False, False, 1.0, True, True, p, 4, 0, 0) == 10            # valid correction: unsupported
    assert f(p, p, 0, 2, 2, 2, False, False, 1.0, True, True, None, 0, 0, 0) == 0          # empty batch
    assert f(p, p, 1, 100, 2, 100, False, False, 1.0, True, True, None, 0, 0, 0) == 10     # size overflow
    # degrees beyond 64 are refused while the arguments are checked, as in the reference (nothing is launched)
    assert f(p, p, 1, 2, 2, 62, False, True, 1.0, True, True, None, 0, 0, 0) == 10         # 4 channels: length overflows
    assert f(p, p, 1, 2, 2, 65, False, False, 1.0, True, True, None, 0, 0, 0) == 10        # 2^66 coefficients: overflows first
    bp = L.CUSIG_SIG_BACKPROP["float64"]
    assert f(p, p, 1, 1, 2, 70, True, False, 1.0, True, True, None, 0, 0, 0) == 10         # time-augmented: 2 channels
    assert f(p, p, 1, 2, 2, 60, False, False, 1.0, True, True, None, 0, 0, 0) == 10        # 2^61 coefficients: no launch possible
    assert "too large" in L.last_error_message()
    assert bp(p, p, p, p, 1, 5, 2, 17, False, False, 1.0, True, None, 0, 0, 0) == 10       # 5 channels, degree 17: no kernel
    assert "no kernel" in L.last_error_message()
    # degree 17 of two channels is served (a path that does not move has the zero signature)
    assert not P.sig(torch.zeros(1, 3, 2, dtype=torch.float64, device=DEV), 17).any()
    y = torch.zeros(3, 4, 2, dtype=torch.float64, device=DEV)
    with pytest.raises(ValueError):                                   # width matches neither convention
        P.sig_backprop(y, torch.zeros(3, 5, dtype=torch.float64, device=DEV),
                       torch.zeros(3, 5, dtype=torch.float64, device=DEV), 2)
    with pytest.raises(ValueError):                                   # dtype mismatch
        P.sig_backprop(y, torch.zeros(3, 6, dtype=torch.float32, device=DEV),
                       torch.zeros(3, 6, dtype=torch.float32, device=DEV), 2)
    with pytest.raises(ValueError):                                   # batch mismatch
        P.sig_backprop(y, torch.zeros(2, 6, dtype=torch.float64, device=DEV),
                       torch.zeros(2, 6, dtype=torch.float64, device=DEV), 2)


def test_autograd_wrapper(P, oracle):
    rng = np.random.default_rng(8)
    for aug in ({}, dict(time_aug=True, lead_lag=True, end_time=2.0)):
        x = rng.standard_normal((3, 9, 3))
        ref = oracle.signature(x, 4, **aug)
        g = rng.standard_normal(ref.shape)
        ref_b = oracle.sig_backprop(x, ref, g, 4, **aug)
        xt = dev(x).requires_grad_()
        out = P.torch_api.sig(xt, 4, **aug)
        (grad,) = torch.autograd.grad(out, xt, dev(g))
        np.testing.assert_allclose(out.detach().cpu().numpy(), ref, rtol=1e-11, atol=1e-12)
        np.testing.assert_allclose(grad.cpu().numpy(), ref_b, rtol=1e-10, atol=1e-11)
    # finite-difference directional derivative (tests/test_cuda_horner.py:131-146 of the reference)
    x = dev(rng.standard_normal((2, 6, 3))).requires_grad_()
    seeds = dev(rng.standard_normal((2, 120)))
    direction = dev(rng.standard_normal((2, 6, 3)))
    (grad,) = torch.autograd.grad(P.torch_api.sig(x, 4), x, seeds)
    eps = 1e-5
    fd = ((P.sig(x.detach() + eps * direction, 4) - P.sig(x.detach() - eps * direction, 4)) * seeds).sum() / (2 * eps)
    torch.testing.assert_close((grad * direction).sum(), fd, atol=2e-7, rtol=2e-7)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_inputs_from_a_side_stream(P, oracle, dtype, scalar_term):
    """Inputs produced, and results consumed, on a non-default stream (a non-contiguous batch view, as in
    tests/test_cuda_horner.py:149-167 of the reference): the entry points wait for the device on entry, so work
    queued on any stream is seen, and they return with their own work done."""
    rng = np.random.default_rng(98)
    data = (0.025 * np.cumsum(rng.standard_normal((2, 2, 131, 6)), axis=-2)).astype(dtype)
    x = np.ascontiguousarray(data[..., ::2])
    flat = x.reshape(4, 131, 3)
    want = oracle.signature(flat, 10, scalar_term=scalar_term, n_jobs=-1)
    seeds = (0.03 * rng.standard_normal(want.shape)).astype(dtype)
    want_grad = oracle.sig_backprop(flat, want, seeds, 10, n_jobs=-1)
    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        # a chain of kernels on the side stream right before the call: the call must not start ahead of them
        staged = torch.tensor(data, device=DEV)
        for _ in range(20):
            staged = staged * 1.0 + 0.0
        path = staged[..., ::2].requires_grad_()
        got = P.torch_api.signature(path, 10, scalar_term=scalar_term)
        (grad,) = torch.autograd.grad(got, path, torch.tensor(seeds.reshape(2, 2, -1), device=DEV))
        got_host = (got.detach() * 1.0).cpu().numpy()
        grad_host = (grad * 1.0).cpu().numpy()
    stream.synchronize()
    d_tol = TOL[dtype]
    assert level_rel_err(got_host.reshape(4, -1)[:, (1 if scalar_term else 0):], want[:, (1 if scalar_term else 0):], 3, 10) <= d_tol
    assert bwd_rel_err(grad_host.reshape(4, 131, 3), want_grad) <= d_tol


def test_two_host_threads(P, oracle):
    """The entry points are re-entrant: two host threads calling sig, sig_backprop and the log signature with different
    shapes at the same time get the results of serial calls (the library serialises them on its workspaces; error
    messages and the overflow report are per thread)."""
    import ctypes
    import threading
    from pysiglib_amd import _loader as L
    rng = np.random.default_rng(606)
    jobs = []
    for (b, length, d, deg, dtype) in [(6, 70, 3, 5, np.float64), (3, 33, 10, 4, np.float32), (16, 20, 2, 8, np.float64),
                                       (2, 150, 6, 3, np.float32), (5, 40, 4, 6, np.float64), (4, 64, 12, 3, np.float64)]:
        x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.2).astype(dtype)
        ref = oracle.signature(x, deg, n_jobs=-1)
        g = rng.standard_normal(ref.shape).astype(dtype)
        jobs.append((x, deg, g, ref, oracle.sig_backprop(x, ref, g, deg, n_jobs=-1),
                     oracle.sig_to_log_sig(ref.astype(np.float64), d, deg, 1 if d == 3 else 0)))
    P.prepare_log_sig(3, 5, method=1)
    errors = []

    def worker(which):
        try:
            torch.cuda.set_device(0)
            for rep in range(6):
                for i, (x, deg, g, ref, ref_b, ref_log) in enumerate(jobs):
                    if (i + rep) % 2 != which:
                        continue
                    d = x.shape[2]
                    out = P.sig(dev(x), deg)
                    assert level_rel_err(out.cpu().numpy(), ref, d, deg) <= TOL[x.dtype.type], ("fwd", i)
                    got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
                    assert bwd_rel_err(got_b, ref_b) <= TOL[x.dtype.type], ("bwd", i)
                    if x.dtype == np.float64:
                        got_log = P.sig_to_log_sig(dev(ref), d, deg, method=1 if d == 3 else 0).cpu().numpy()
                        assert np.abs(got_log - ref_log).max() <= 1e-10 * max(1.0, np.abs(ref_log).max()), ("log", i)
                    if d == 3 and which == 0:
                        P.prepare_log_sig(3, 5, method=2 if rep % 2 else 1)     # replaces a table while the other thread runs
                # a failing call leaves its message with the calling thread only
                bad = torch.zeros(8, dtype=torch.float64, device=DEV)
                ptr = ctypes.cast(bad.data_ptr(), ctypes.POINTER(ctypes.c_double))
                if which == 0:
                    assert L.CUSIG_SIGNATURE["float64"](ptr, ptr, 1, 0, 2, 2, False, False, 1.0, True, True, None, 0, 0, 0) == 2
                    assert "dimension 0" in L.last_error_message()
                else:
                    assert L.CUSIG_SIG_BACKPROP["float64"](ptr, ptr, ptr, ptr, 1, 2, 2, 2, False, True, 1.0, True, ptr, 4, 0, 0) == 2
                    assert "lead_lag" in L.last_error_message()
        except BaseException as exc:       # noqa: BLE001 - reported by the main thread
            errors.append((which, repr(exc)))

    threads = [threading.Thread(target=worker, args=(w,)) for w in (0, 1)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not any(t.is_alive() for t in threads)
    assert not errors, errors


def test_reused_buffers_and_repeatability(P, oracle):
    # the library keeps internal workspaces between calls: interleave shapes and repeat
    rng = np.random.default_rng(21)
    cases = [(4, 65, 2, 4), (2, 30, 10, 5), (16, 9, 3, 4), (4, 65, 2, 4)]
    for (b, length, d, deg) in cases * 2:
        x = rng.standard_normal((b, length, d)) * 0.4
        ref = oracle.signature(x, deg, n_jobs=-1)
        g = rng.standard_normal(ref.shape)
        assert level_rel_err(P.sig(dev(x), deg).cpu().numpy(), ref, d, deg) <= 1e-10
        assert bwd_rel_err(P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy(),
                           oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)) <= 1e-10


@pytest.mark.parametrize("segments", [1, 2, 3, 5, 6, 7, 8, 11, 13, 32])
def test_time_segmented_forward(P, oracle, segments):
    """The forward sweep may split paths into time segments folded with Chen's identity; every split must agree."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    rng = np.random.default_rng(40 + segments)
    cases = [((3, 17, 3, 4), {}, False), ((2, 64, 10, 5), {}, True), ((2, 9, 2, 6), dict(time_aug=True, lead_lag=True), False),
             ((5, 4, 6, 3), {}, True), ((1, 100, 5, 7), {}, False), ((70, 23, 2, 3), dict(lead_lag=True), True)]
    try:
        L.CUSIG.cusig_amd_force_segments(segments)
        for (shape, aug, scalar_term) in cases:
            b, length, d, deg = shape
            for dtype in (np.float64, np.float32):
                x = (rng.standard_normal(shape[:3]) * 0.4).astype(dtype)
                ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1, **aug)
                got = P.sig(dev(x), deg, scalar_term=scalar_term, **aug).cpu().numpy()
                off = 1 if scalar_term else 0
                d_aug = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
                if scalar_term:
                    np.testing.assert_array_equal(got[:, 0], 1.0)
                assert level_rel_err(got[:, off:], ref[:, off:], d_aug, deg) <= TOL[dtype], (shape, aug, dtype)
    finally:
        L.CUSIG.cusig_amd_force_segments(0)


@pytest.mark.parametrize("segments", [2, 3, 7, 16])
def test_time_segmented_backward(P, oracle, segments):
    """The backward sweep may be cut in time too (states from running Chen products of the segment signatures,
    adjoints from the product's pullback); every split must give the whole-path gradient."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_bwd_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_bwd_segments.restype = None
    rng = np.random.default_rng(140 + segments)
    cases = [((3, 41, 3, 4), {}, False),                                  # a few paths per wave
             ((2, 64, 10, 5), {}, True),                                  # wide layout, paired reduction in f64
             ((2, 33, 2, 6), dict(time_aug=True, lead_lag=True), False),
             ((5, 18, 6, 3), {}, True),
             ((1, 100, 5, 7), {}, False),
             ((70, 23, 2, 3), dict(lead_lag=True), True),                 # many paths per wave, ragged last segment
             ((9, 50, 2, 2), {}, False),
             ((2, 40, 20, 3), {}, False),                                 # run-time-dimension kernel
             ((2, 37, 40, 2), {}, True),                                  # too wide for the reduction tile
             ((3, 130, 6, 4), dict(time_aug=True), False)]
    try:
        L.CUSIG.cusig_amd_force_bwd_segments(segments)
        for (shape, aug, scalar_term) in cases:
            b, length, d, deg = shape
            for dtype in (np.float64, np.float32):
                x = (np.cumsum(rng.standard_normal(shape[:3]), axis=1) * (0.8 / np.sqrt(length))).astype(dtype)
                ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1, **aug)
                g = rng.standard_normal(ref.shape).astype(dtype)
                want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, **aug)
                got = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
                assert bwd_rel_err(got, want) <= TOL[dtype], (shape, aug, dtype, bwd_rel_err(got, want))
    finally:
        L.CUSIG.cusig_amd_force_bwd_segments(0)


@pytest.mark.parametrize("shape,dtype", [
    ((2, 5, 98, 2), np.float64), ((2, 4, 350, 2), np.float32), ((1, 3, 1000, 2), np.float64),     # wide paths, low degree
    ((70000, 3, 2, 2), np.float32), ((66000, 4, 3, 3), np.float64),                                # batch beyond 65535
    ((3, 2000, 2, 4), np.float64), ((1, 20001, 3, 3), np.float64),                                 # long paths
    ((1, 100000, 3, 6), np.float64), ((1, 65536, 2, 10), np.float64), ((2, 16000, 5, 5), np.float64),      # hundreds of time pieces
    ((2, 6, 2, 16), np.float64), ((1, 4, 3, 11), np.float64),                                      # highest compiled degrees
    ((2, 6, 2, 20), np.float64), ((1, 5, 2, 24), np.float64), ((1, 4, 3, 17), np.float64),         # run-time-degree sweeps
    ((2, 5, 2, 18), np.float32),
])
def test_extreme_shapes(P, oracle, shape, dtype):
    """Shapes the reference's GPU suite probes for its launch and memory limits
    (tests/test_signature_cuda_shared_memory.py, tests/test_cuda_grid_limits.py of the reference)."""
    b, length, d, deg = shape
    rng = np.random.default_rng(b + length + d + deg)
    scale = 1.0 / np.sqrt(length) if length > 100 else 0.5
    x = np.cumsum(rng.standard_normal((b, length, d)) * scale, axis=1).astype(dtype)
    ref = oracle.signature(x, deg, n_jobs=-1)
    got = P.sig(dev(x), deg).cpu().numpy()
    assert level_rel_err(got, ref, d, deg) <= TOL[dtype]
    g = rng.standard_normal(ref.shape).astype(dtype)
    ref_b = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
    got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
    assert bwd_rel_err(got_b, ref_b) <= TOL[dtype]


@pytest.mark.parametrize("shape,aug,scalar_term", [
    ((1, 5, 64, 4), {}, False),                                     # one tile of 64 prefixes x 64 letters per word row
    ((2, 6, 49, 4), {}, True), ((2, 4, 52, 4), dict(time_aug=True), False),       # partly filled tiles
    ((2, 5, 70, 4), {}, False), ((1, 4, 130, 3), {}, True),         # several tiles per row; degree 3 beyond the table
    ((1, 3, 300, 3), {}, False), ((3, 2, 64, 3), {}, True),         # 5 x 5 (10 in double precision) tiles per row; a single step
    ((3, 6, 25, 4), dict(lead_lag=True, time_aug=True), False),     # 51 augmented channels
    ((2, 4, 33, 5), {}, False),                                     # chains of four letters
])
def test_by_row_reverse_sweep(P, oracle, shape, aug, scalar_term):
    """Backward of many channels where the compiled table has no faster kernel (sig_rows.hip), both precisions, against
    the oracle; and the general run-time kernels on the same input (hook off) as a second opinion on the dispatch."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_rows_backward.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_rows_backward.restype = None
    L.CUSIG.cusig_amd_set_rows_forward.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_rows_forward.restype = None
    L.CUSIG.cusig_amd_last_kernel_name.restype = ctypes.c_char_p
    b, length, d, deg = shape
    rng = np.random.default_rng(b * 100000 + length * 1000 + d * 10 + deg)
    x64 = np.cumsum(rng.standard_normal((b, length, d)), axis=1) * (1.5 / np.sqrt(d))
    for dtype in (np.float32, np.float64):
        x = x64.astype(dtype)
        ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1, **aug)
        g = rng.standard_normal(ref.shape).astype(dtype)
        want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, **aug)
        d_aug = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
        off = 1 if scalar_term else 0
        try:
            L.CUSIG.cusig_amd_set_profiling(1)
            # the forward sweep in the same tiling, where the shape has no compiled forward instance
            fwd = P.sig(dev(x), deg, scalar_term=scalar_term, **aug).cpu().numpy()
            name = L.CUSIG.cusig_amd_last_kernel_name().decode()
            compiled = (deg == 3 and d_aug <= 128) or (deg == 4 and d_aug <= 48)
            if not compiled and (dtype == np.float64 or d_aug % 32):
                assert name == "rows_fwd_%s_n%d" % ("f32" if dtype == np.float32 else "f64", deg), name
            assert L.CUSIG.cusig_amd_last_sig_nonfinite() == 0
            if scalar_term:
                np.testing.assert_array_equal(fwd[:, 0], 1.0)
            assert level_rel_err(fwd[:, off:], ref[:, off:], d_aug, deg) <= TOL[dtype], (dtype, name)
            L.CUSIG.cusig_amd_set_rows_forward(0)
            fwd_other = P.sig(dev(x), deg, scalar_term=scalar_term, **aug).cpu().numpy()
            assert not L.CUSIG.cusig_amd_last_kernel_name().decode().startswith("rows_fwd")
            np.testing.assert_array_equal(fwd_other, fwd)       # the same arithmetic in the same order
            got = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
            assert L.CUSIG.cusig_amd_last_kernel_name().decode() == "rows_bwd_%s_n%d" % ("f32" if dtype == np.float32 else "f64", deg)
            L.CUSIG.cusig_amd_set_rows_backward(0)
            other = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
            assert not L.CUSIG.cusig_amd_last_kernel_name().decode().startswith("rows_bwd")
        finally:
            L.CUSIG.cusig_amd_set_rows_backward(1)
            L.CUSIG.cusig_amd_set_rows_forward(1)
            L.CUSIG.cusig_amd_set_profiling(0)
        assert bwd_rel_err(got, want) <= TOL[dtype], (dtype, bwd_rel_err(got, want))
        assert bwd_rel_err(other, want) <= TOL[dtype], (dtype, bwd_rel_err(other, want))


@pytest.mark.parametrize("shape", [(3, 9, 2, 5), (2, 7, 2, 9), (5, 12, 2, 12), (2, 6, 3, 4), (3, 10, 3, 7), (2, 9, 3, 10),
                                   (4, 8, 4, 3), (2, 11, 4, 6), (70, 5, 2, 6), (1, 300, 3, 5)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_run_time_degree_sweeps(P, oracle, shape, dtype):
    """The sweeps that serve degrees 17 .. 64 (2 to 4 augmented channels, chain of run-time length in LDS), forced onto
    small shapes: against the oracle, forward and backward, plain and augmented paths, with and without scalar term."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_deep.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_deep.restype = None
    b, length, d, deg = shape
    rng = np.random.default_rng(b * 1000 + d * 10 + deg)
    x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * (0.3 if length < 100 else 0.05)).astype(dtype)
    L.CUSIG.cusig_amd_force_deep(1)
    try:
        ref = oracle.signature(x, deg, n_jobs=-1)
        g = rng.standard_normal(ref.shape).astype(dtype)
        got = P.sig(dev(x), deg)
        assert level_rel_err(got.cpu().numpy(), ref, d, deg) <= TOL[dtype]
        assert L.CUSIG.cusig_amd_last_kernel_name is not None
        got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
        assert bwd_rel_err(got_b, oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)) <= TOL[dtype]
        with_scalar = P.sig(dev(x), deg, scalar_term=True).cpu().numpy()
        assert np.all(with_scalar[:, 0] == 1) and np.array_equal(with_scalar[:, 1:], got.cpu().numpy())
        if d == 2 and deg <= 6:
            # one raw channel with time: 2 augmented channels; with lead-lag and time: 3
            x1 = x[:, :, :1].copy()
            for aug in (dict(time_aug=True, end_time=0.7), dict(time_aug=True, lead_lag=True)):
                ref = oracle.signature(x1, deg, **aug)
                d_aug = 2 + (1 if aug.get("lead_lag") else 0)
                assert level_rel_err(P.sig(dev(x1), deg, **aug).cpu().numpy(), ref, d_aug, deg) <= TOL[dtype]
                g = rng.standard_normal(ref.shape).astype(dtype)
                want = oracle.sig_backprop(x1, ref, g, deg, **aug)
                assert bwd_rel_err(P.sig_backprop(dev(x1), dev(ref), dev(g), deg, **aug).cpu().numpy(), want) <= TOL[dtype]
    finally:
        L.CUSIG.cusig_amd_force_deep(0)


@pytest.mark.parametrize("shape", [
    (3, 9, 13, 4), (2, 12, 20, 3), (5, 7, 30, 2), (2, 6, 32, 3), (3, 8, 50, 2), (4, 9, 40, 2), (2, 5, 18, 5), (2, 6, 100, 2),
    (70, 5, 12, 2), (2, 7, 27, 3), (2, 6, 33, 3), (1, 30, 64, 2),
    (2, 6, 70, 3), (1, 5, 34, 4), (2, 5, 17, 5), (3, 40, 65, 3),
    (2, 6, 130, 3), (2, 7, 97, 3), (1, 5, 41, 4), (2, 5, 21, 5), (1, 4, 200, 3),        # beyond the specialised table: run-time dimension
    (1, 4, 48, 4), (1, 3, 24, 5), (2, 5, 9, 6), (2, 6, 10, 6), (1, 4, 12, 6), (1, 4, 6, 7), (1, 4, 7, 7), (1, 4, 8, 7),
    (1, 4, 5, 8), (1, 3, 6, 8), (1, 3, 4, 9), (1, 3, 4, 10), (1, 4, 13, 6), (1, 3, 9, 7), (1, 3, 5, 9), (1, 3, 7, 8), (1, 4, 49, 4), (1, 3, 25, 5)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_many_channel_shapes(P, oracle, shape, dtype):
    """Dimensions beyond the specialised instances run the run-time-dimension kernels, which come in several
    letter counts per lane and two lane layouts: every one of them against the oracle, forward and backward,
    whole paths and time-split sweeps."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_bwd_segments.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_bwd_segments.restype = None
    b, length, d, deg = shape
    rng = np.random.default_rng(b * 1000 + d * 10 + deg)
    x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.3).astype(dtype)
    ref = oracle.signature(x, deg, n_jobs=-1)
    g = rng.standard_normal(ref.shape).astype(dtype)
    want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
    try:
        for segments in (0, 2):
            L.CUSIG.cusig_amd_force_segments(segments)
            L.CUSIG.cusig_amd_force_bwd_segments(segments)
            got = P.sig(dev(x), deg).cpu().numpy()
            assert level_rel_err(got, ref, d, deg) <= TOL[dtype], (shape, segments)
            got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
            assert bwd_rel_err(got_b, want) <= TOL[dtype], (shape, segments)
    finally:
        L.CUSIG.cusig_amd_force_segments(0)
        L.CUSIG.cusig_amd_force_bwd_segments(0)
    xa = x[:, :, : min(d, 23)]
    aug = dict(time_aug=True, lead_lag=(d <= 25))
    refa = oracle.signature(xa, min(deg, 3), n_jobs=-1, **aug)
    da = (2 * xa.shape[2] if aug["lead_lag"] else xa.shape[2]) + 1
    assert level_rel_err(P.sig(dev(xa), min(deg, 3), **aug).cpu().numpy(), refa, da, min(deg, 3)) <= TOL[dtype]


@pytest.mark.parametrize("shape", [(1, 5, 49, 4), (1, 4, 52, 4), (1, 4, 25, 5), (1, 5, 13, 6), (1, 4, 9, 7), (1, 3, 7, 8),
                                   (1, 3, 6, 9), (1, 3, 5, 10)])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_every_run_time_dimension_variant(P, oracle, shape, dtype):
    """The run-time-dimension kernels exist with 4 letters per lane in the packed layout for every degree and, up to
    degree 10 (backward: 8), with 8, 16 or 32 letters per lane in the packed or the wide layout; the choice among them follows the
    channel count.  Here every compiled variant of a degree is forced onto one shape (letter groups that fill the row
    exactly, reach past it, or hold it in one partly empty group) and checked against the oracle in both directions."""
    import ctypes
    from pysiglib_amd import _loader as L
    C = L.CUSIG
    C.cusig_amd_force_partition.argtypes = (ctypes.c_int, ctypes.c_int)
    C.cusig_amd_force_partition.restype = None
    C.cusig_amd_force_run_time_wide.argtypes = (ctypes.c_int,)
    C.cusig_amd_force_run_time_wide.restype = None
    b, length, d, deg = shape
    if deg <= 5:
        variants = {False: [(0, 4), (1, 16), (1, 32)], True: [(0, 4), (0, 16), (1, 16), (1, 32)]}
    elif deg <= 8:
        variants = {False: [(0, 4), (1, 8), (1, 16)], True: [(0, 4), (0, 16), (1, 8), (1, 16)]}
    else:
        variants = {False: [(0, 4), (1, 8)], True: [(0, 4)]}
    rng = np.random.default_rng(d * 100 + deg)
    x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.3).astype(dtype)
    ref = oracle.signature(x, deg, n_jobs=-1)
    g = rng.standard_normal(ref.shape).astype(dtype)
    want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
    try:
        C.cusig_amd_set_profiling(1)
        for backward in (False, True):
            for (wide, k) in variants[backward]:
                C.cusig_amd_force_run_time_wide(wide)
                C.cusig_amd_force_partition(1, k)
                if backward:
                    got = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
                else:
                    got = P.sig(dev(x), deg).cpu().numpy()
                name = C.cusig_amd_last_kernel_name().decode()
                assert ("_d0w_" if wide else "_d0_") in name and name.endswith("_t1_k%d" % k), (name, wide, k)
                if backward:
                    assert bwd_rel_err(got, want) <= TOL[dtype], (shape, name)
                else:
                    assert level_rel_err(got, ref, d, deg) <= TOL[dtype], (shape, name)
    finally:
        C.cusig_amd_force_partition(0, 0)
        C.cusig_amd_force_run_time_wide(0)
        C.cusig_amd_set_profiling(0)


@pytest.mark.parametrize("shape,aug", [
    ((3, 9, 2), {}), ((2, 30, 5), {}), ((4, 17, 16), dict(time_aug=True)), ((2, 21, 17), dict(lead_lag=True)),
    ((3, 12, 33), dict(time_aug=True, lead_lag=True)), ((2, 2, 70), {}), ((2, 40, 64), {}), ((3, 25, 80), {}),
    ((1, 9, 130), dict(time_aug=True)), ((1, 6, 256), {}), ((70, 5, 65), {}), ((70000, 3, 2), {})])      # the last: more paths than a grid dimension holds
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_degree_three_matrix_form(P, oracle, shape, aug, dtype, scalar_term):
    """Degree 3 as library matrix products around a scan (forward: one product, backward: two), forced onto narrow
    paths too, against the oracle; the sweep kernels' backward on the same inputs beside it."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_degree3.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_degree3.restype = None
    b, length, d = shape
    rng = np.random.default_rng(b * 1000 + d * 10 + length)
    # The 70000 two-step paths get a drift: among that many driftless ones some nearly close, their level 3 cancels to
    # 1e-6 and every float32 evaluation (the oracle's included) is then 2-3e-4 off the float64 value.
    drift = 1.0 if b > 60000 else 0.0
    x = (np.cumsum(rng.standard_normal((b, length, d)) * 0.3 + drift, axis=1)).astype(dtype)
    ref = oracle.signature(x, 3, n_jobs=-1, scalar_term=scalar_term, **aug)
    g = rng.standard_normal(ref.shape).astype(dtype)
    want = oracle.sig_backprop(x, ref, g, 3, n_jobs=-1, **aug)
    try:
        L.CUSIG.cusig_amd_force_degree3(1)
        fwd = P.sig(dev(x), 3, scalar_term=scalar_term, **aug).cpu().numpy()
        assert L.CUSIG.cusig_amd_last_sig_nonfinite() == 0
        got = P.sig_backprop(dev(x), dev(ref), dev(g), 3, **aug).cpu().numpy()
        L.CUSIG.cusig_amd_force_degree3(0)
        sweep = P.sig_backprop(dev(x), dev(ref), dev(g), 3, **aug).cpu().numpy()
    finally:
        L.CUSIG.cusig_amd_force_degree3(-1)
    d_aug = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    off = 1 if scalar_term else 0
    assert level_rel_err(fwd[:, off:], ref[:, off:], d_aug, 3) <= TOL[dtype], shape
    if scalar_term:
        assert np.all(fwd[:, 0] == 1)
    assert bwd_rel_err(got, want) <= TOL[dtype], shape
    assert bwd_rel_err(sweep, want) <= TOL[dtype], shape


@pytest.mark.parametrize("dtype", ["float64", "float32"])
def test_degree_two_pointers_aligned_to_the_element_only(dtype):
    """The C ABI promises nothing beyond element alignment: the degree-2 kernels that copy rows in 16-byte pieces must
    fall back to element-wise copies for such pointers and return the same bits."""
    import ctypes
    from pysiglib_amd import _loader as L
    tdt = torch.float64 if dtype == "float64" else torch.float32
    real = L.DTYPES[dtype]
    b, length, d = 9, 70, 64
    n = d + d * d
    gen = torch.Generator(device="cpu").manual_seed(5)
    x = (torch.randn((b, length, d), dtype=tdt, generator=gen).cumsum(1) * 0.05).to(DEV)
    g = torch.randn((b, n), dtype=tdt, generator=gen).to(DEV)
    esz = x.element_size()
    res = []
    for shift in (0, 1):
        xs = torch.zeros(x.numel() + 4, dtype=tdt, device=DEV)
        xs[shift:shift + x.numel()] = x.flatten()
        gs = torch.zeros(g.numel() + 4, dtype=tdt, device=DEV)
        gs[shift:shift + g.numel()] = g.flatten()
        sig = torch.zeros(b * n + 4, dtype=tdt, device=DEV)
        gx = torch.zeros(x.numel() + 4, dtype=tdt, device=DEV)
        ptr = lambda t: ctypes.cast(t.data_ptr() + shift * esz, ctypes.POINTER(real))
        assert L.CUSIG_SIGNATURE[dtype](ptr(xs), ptr(sig), b, d, length, 2, False, False, 1.0, True, False, None, 0, 0, 0) == 0
        assert L.CUSIG_SIG_BACKPROP[dtype](ptr(xs), ptr(gx), ptr(gs), ptr(sig), b, d, length, 2, False, False, 1.0, False,
                                           None, 0, 0, 0) == 0
        res.append((sig[shift:shift + b * n].clone(), gx[shift:shift + x.numel()].clone()))
    assert torch.equal(res[0][0], res[1][0]) and torch.equal(res[0][1], res[1][1])
    assert float(res[0][0].abs().max()) > 0 and float(res[0][1].abs().max()) > 0


@pytest.mark.parametrize("shape,aug", [
    ((3, 9, 2, 2), {}), ((2, 30, 5, 2), {}), ((4, 17, 16, 2), {}), ((2, 21, 17, 2), dict(time_aug=True)),
    ((2, 13, 31, 2), dict(lead_lag=True)), ((3, 12, 33, 2), dict(time_aug=True, lead_lag=True)), ((1, 2, 70, 2), {}),
    ((2, 700, 20, 2), {}),                      # few long paths: time slices adding into the output
    ((2, 600, 50, 2), {}), ((1, 300, 36, 2), dict(lead_lag=True)),      # the same with operands staged through LDS
    ((1, 1500, 7, 2), dict(lead_lag=True)), ((70, 6, 65, 2), {}), ((2, 5, 130, 2), dict(time_aug=True)),
    ((3, 300, 64, 2), {}), ((2, 41, 128, 2), {}), ((2, 150, 100, 2), {}), ((5, 3, 64, 2), {}),      # rows in 16-byte pieces
    ((2, 100, 40, 2), dict(time_aug=True)), ((3, 70, 33, 2), {}), ((1, 1000, 48, 2), {}), ((4, 2, 56, 2), {})])
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_degree_two_closed_form(P, oracle, shape, aug, dtype):
    """Degree 2 has a closed form in the path (S2 = U^T Z, pullback through the antisymmetric part of the level-2
    gradient) that runs on the matrix cores; forced on for every dimension here and compared with the oracle's sweep."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_force_degree2.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_degree2.restype = None
    b, length, d, deg = shape
    rng = np.random.default_rng(b * 1000 + d * 10 + length)
    x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * (1.0 / np.sqrt(length))).astype(dtype)
    d_aug = (2 * d if aug.get("lead_lag") else d) + (1 if aug.get("time_aug") else 0)
    L.CUSIG.cusig_amd_set_degree2_staged.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_degree2_staged.restype = None
    try:
        # forced on (operands staged through LDS where that applies, then straight from memory), then forced off
        # (the sweep kernels of degree 2 stay covered)
        for mode, scalar_term, staged in ((1, False, 1), (1, True, 0), (0, True, 1)):
            L.CUSIG.cusig_amd_force_degree2(mode)
            L.CUSIG.cusig_amd_set_degree2_staged(staged)
            ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1, **aug)
            off = 1 if scalar_term else 0
            with warnings.catch_warnings():
                warnings.simplefilter("error", RuntimeWarning)       # a finite result must not be reported as overflow
                got = P.sig(dev(x), deg, scalar_term=scalar_term, **aug).cpu().numpy()
            if scalar_term:
                np.testing.assert_array_equal(got[:, 0], 1.0)
            assert level_rel_err(got[:, off:], ref[:, off:], d_aug, deg) <= TOL[dtype], (shape, aug, scalar_term)
            g = rng.standard_normal(ref.shape).astype(dtype)
            want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, **aug)
            got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
            assert bwd_rel_err(got_b, want) <= TOL[dtype], (shape, aug, scalar_term)
        big = x.copy()
        big[0] *= 1e200 if dtype == np.float64 else 1e30
        with pytest.warns(RuntimeWarning):
            P.sig(dev(big), deg, **aug)
    finally:
        L.CUSIG.cusig_amd_force_degree2(-1)
        L.CUSIG.cusig_amd_set_degree2_staged(1)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_every_specialised_dimension_above_12(P, oracle, dtype):
    """One small forward + backward per compiled (dimension, degree) instance that the grid above does not reach
    (backward: up to 47 channels, beyond which the by-row reverse sweep takes over):
    dimensions 13..64 at degree 3, 13..32 and 41..48 at degree 4, 9..16 and 21..24 at degree 5, 7..12 at degree 6, 6..8 at degree 7, 5..6 at
    degree 8, 4..5 at degree 9, 4 at degree 10, 2 at degrees 13..16, 3 at degrees 13 and 14."""
    import ctypes
    from pysiglib_amd import _loader as L
    C = L.CUSIG
    C.cusig_amd_force_partition.argtypes = (ctypes.c_int, ctypes.c_int)
    C.cusig_amd_force_partition.restype = None
    rng = np.random.default_rng(5)
    shapes = ([(d, 3) for d in range(13, 65)] + [(d, 4) for d in range(13, 33)] + [(d, 4) for d in range(41, 49)] +
              [(d, 5) for d in range(9, 17)] + [(d, 5) for d in range(21, 25)] +
              [(7, 6), (8, 6), (9, 6), (10, 6), (11, 6), (12, 6), (6, 7), (7, 7), (8, 7), (5, 8), (6, 8), (4, 9), (5, 9), (4, 10),
               (2, 13), (2, 14), (2, 15), (2, 16), (3, 13), (3, 14)])
    tail, k, spec = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()

    def pin(backward, d, deg):
        # tiny batches would be handed to the run-time-dimension kernel: pin the instance's own partition
        C.cusig_amd_force_partition(0, 0)
        assert C.cusig_amd_kernel_choice(int(backward), int(dtype == np.float64), d, deg, tail, k, spec) == 1
        assert spec.value == 1, (d, deg)
        C.cusig_amd_force_partition(tail.value, k.value)

    try:
        C.cusig_amd_set_profiling(1)
        for (d, deg) in shapes:
            b, length = (2, 4) if d ** deg < 200000 else (1, 3)
            x = (rng.standard_normal((b, length, d)) * 0.5).astype(dtype)
            ref = oracle.signature(x, deg, n_jobs=-1)
            pin(False, d, deg)
            got = P.sig(dev(x), deg).cpu().numpy()
            assert ("_d%d_n%d_" % (d, deg)) in C.cusig_amd_last_kernel_name().decode()
            assert level_rel_err(got, ref, d, deg) <= TOL[dtype], (d, deg)
            g = rng.standard_normal(ref.shape).astype(dtype)
            want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
            if d >= 48:
                # from 48 channels on the backward has no compiled instance: the by-row reverse sweep serves it
                C.cusig_amd_force_partition(0, 0)
            else:
                pin(True, d, deg)
            got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg).cpu().numpy()
            name = C.cusig_amd_last_kernel_name().decode()
            assert name.startswith("rows_bwd_") if d >= 48 else ("_d%d_n%d_" % (d, deg)) in name, (d, deg, name)
            assert bwd_rel_err(got_b, want) <= TOL[dtype], (d, deg)
    finally:
        C.cusig_amd_force_partition(0, 0)
        C.cusig_amd_set_profiling(0)


def test_randomised_shapes(P, oracle):
    """400 seeded random draws over the whole instance table: dimension, degree, batch, length, augmentations,
    dtype, scalar term and forced time splits of both sweeps, each against the oracle."""
    import ctypes
    from pysiglib_amd import _loader as L
    C = L.CUSIG
    C.cusig_amd_force_segments.argtypes = (ctypes.c_int,)
    C.cusig_amd_force_bwd_segments.argtypes = (ctypes.c_int,)
    C.cusig_amd_force_bwd_segments.restype = None
    caps = {2: 12, 3: 12, 4: 8, 5: 7, 6: 6, 7: 6, 8: 6}
    caps.update({d: 5 for d in range(9, 17)})
    caps.update({d: 4 for d in range(17, 33)})
    caps.update({d: 3 for d in range(33, 70)})
    rng = np.random.default_rng(2024)
    try:
        for it in range(400):
            time_aug, lead_lag = bool(rng.integers(0, 4) == 0), bool(rng.integers(0, 4) == 0)
            d = int(rng.choice(list(caps.keys())))
            if lead_lag:
                d = max(1, d // 2)
            d_aug = (2 * d if lead_lag else d) + (1 if time_aug else 0)
            deg = int(rng.integers(2, caps.get(d_aug, 3) + 1))
            while d_aug ** deg > 3_000_000 and deg > 2:
                deg -= 1
            b = int(rng.choice([1, 2, 3, 5, 17, 70]))
            length = int(rng.choice([2, 3, 5, 9, 33, 70, 131, 300]))
            if d_aug ** deg * b * length > 60_000_000:
                b, length = 1, min(length, 5)
            dtype = np.float64 if rng.integers(0, 2) else np.float32
            scalar_term = bool(rng.integers(0, 2))
            segments = int(rng.choice([0, 0, 2, 3, 5]))
            case = (it, b, length, d, deg, np.dtype(dtype).name, time_aug, lead_lag, scalar_term, segments)
            x = (np.cumsum(rng.standard_normal((b, length, d)), axis=1) * (0.7 / np.sqrt(length))).astype(dtype)
            aug = dict(time_aug=time_aug, lead_lag=lead_lag)
            ref = oracle.signature(x, deg, scalar_term=scalar_term, n_jobs=-1, **aug)
            g = rng.standard_normal(ref.shape).astype(dtype)
            want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, **aug)
            C.cusig_amd_force_segments(segments)
            C.cusig_amd_force_bwd_segments(segments)
            got = P.sig(dev(x), deg, scalar_term=scalar_term, **aug).cpu().numpy()
            got_b = P.sig_backprop(dev(x), dev(ref), dev(g), deg, **aug).cpu().numpy()
            off = 1 if scalar_term else 0
            if scalar_term:
                np.testing.assert_array_equal(got[:, 0], 1.0)
            assert level_rel_err(got[:, off:], ref[:, off:], d_aug, deg) <= TOL[dtype], case
            assert bwd_rel_err(got_b, want) <= TOL[dtype], case
    finally:
        C.cusig_amd_force_segments(0)
        C.cusig_amd_force_bwd_segments(0)


def test_wide_degree_one(P):
    x = torch.randn(3, 2, 200000, dtype=torch.float32, device=DEV)
    torch.testing.assert_close(P.sig(x, 1), x[:, 1] - x[:, 0])
    g = torch.randn(3, 200000, dtype=torch.float32, device=DEV)
    grad = P.sig_backprop(x, P.sig(x, 1), g, 1)
    torch.testing.assert_close(grad[:, 1], g)
    torch.testing.assert_close(grad[:, 0], -g)


# ---- the benchmark workloads at full size -----------------------------------------------------------------

@pytest.mark.parametrize("k", [1, 2, 4])
def test_config_forward_full_size(P, oracle, k):
    c = C.CONFIGS[k]
    x = C.make_path(k)
    kw = dict(time_aug=c["time_aug"], lead_lag=c["lead_lag"], end_time=1.0)
    ref = oracle.signature(x, c["degree"], n_jobs=-1, **kw)
    got = P.sig(dev(x), c["degree"], **kw).cpu().numpy()
    assert got.shape == ref.shape
    assert level_rel_err(got, ref, C.aug_dim(c), c["degree"]) <= TOL[np.dtype(c["dtype"]).type]


def test_config3_forward(P, oracle):
    """(64, 4096, 3) degree 12: every one of the 64 paths against the oracle, and on top of that the size-independent
    properties: level 1 = total increment, the level-2 shuffle identity, batch invariance up to rounding, and Chen's
    identity on every coefficient (the signatures of the two halves of each path, multiplied with the oracle-checked
    Chen product, give the signature of the whole path)."""
    c = C.CONFIGS[3]
    x = C.make_path(3)
    xt = dev(x)
    got = P.sig(xt, 12)
    assert got.shape == (64, 797160)
    ref = oracle.signature(x, 12, n_jobs=-1)
    assert level_rel_err(got.cpu().numpy(), ref, 3, 12) <= 1e-10
    del ref
    l1 = got[:, :3].cpu().numpy()
    np.testing.assert_allclose(l1, x[:, -1] - x[:, 0], rtol=1e-12, atol=1e-14)
    l2 = got[:, 3:12].cpu().numpy().reshape(64, 3, 3)
    np.testing.assert_allclose(l2 + l2.transpose(0, 2, 1), l1[:, :, None] * l1[:, None, :], rtol=1e-10, atol=1e-13)
    # a smaller batch may be cut into time segments (a different order of additions): equal up to rounding
    again = P.sig(xt[40:47].clone(), 12)
    assert level_rel_err(again.cpu().numpy(), got[40:47].cpu().numpy(), 3, 12) <= 1e-12
    del again
    first, second = P.sig(xt[:, :2049].contiguous(), 12), P.sig(xt[:, 2048:].contiguous(), 12)
    whole = P.sig_combine(first, second, 3, 12)
    del first, second
    lo = 0
    for level in range(1, 13):
        a, b = whole[:, lo:lo + 3 ** level], got[:, lo:lo + 3 ** level]
        err = ((a - b).abs().amax(dim=1) / b.abs().amax(dim=1).clamp_min(1e-300)).max().item()
        assert err <= 1e-10, (level, err)
        lo += 3 ** level
    del got, whole
    torch.cuda.empty_cache()


def test_config5_backward_full_size(P, oracle):
    c = C.CONFIGS[5]
    x = C.make_path(5)
    sig = oracle.signature(x, 5, n_jobs=-1)
    g = np.random.default_rng(2005).standard_normal(sig.shape)
    ref = oracle.sig_backprop(x, sig, g, 5, n_jobs=-1)
    got = P.sig_backprop(dev(x), dev(sig), dev(g), 5).cpu().numpy()
    assert bwd_rel_err(got, ref) <= 1e-10
    # linearity in the upstream gradient holds at any size
    got2 = P.sig_backprop(dev(x), dev(sig), dev(2.0 * g), 5).cpu().numpy()
    assert bwd_rel_err(got2, 2.0 * got) <= 1e-12
    # the GPU forward feeds the GPU backward (the autograd pairing)
    sig_gpu = P.sig(dev(x), 5)
    got3 = P.sig_backprop(dev(x), sig_gpu, dev(g), 5).cpu().numpy()
    assert bwd_rel_err(got3, ref) <= 1e-10


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_config4_backward_full_size(P, oracle, dtype):
    """The lead-lag + time workload at its full size through the backward pass (not a benchmark line: the backward
    of an augmented path takes the lead-lag-aware sweep and the fold-back onto the raw points)."""
    c = C.CONFIGS[4]
    x = C.make_path(4).astype(dtype)
    aug = dict(time_aug=True, lead_lag=True)
    sig = oracle.signature(x, c["degree"], n_jobs=-1, **aug)
    g = np.random.default_rng(2004).standard_normal(sig.shape).astype(dtype)
    ref = oracle.sig_backprop(x, sig, g, c["degree"], n_jobs=-1, **aug)
    got = P.sig_backprop(dev(x), dev(sig), dev(g), c["degree"], **aug).cpu().numpy()
    assert got.shape == x.shape
    assert bwd_rel_err(got, ref) <= TOL[dtype]


def test_stream_ordered_mode(P, oracle):
    """Calls that only enqueue on the null stream: results after one synchronisation equal the synchronous ones,
    also when consecutive calls reuse the library's workspaces with different shapes."""
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_stream_ordered.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_set_stream_ordered.restype = None
    rng = np.random.default_rng(99)
    cases = [((6, 50, 4), 4), ((3, 120, 10), 5), ((9, 20, 3), 6), ((2, 300, 2), 3)]
    xs = [dev(rng.standard_normal(shape) * 0.3) for shape, _ in cases]
    want = []
    for x, (_, deg) in zip(xs, cases):
        s = P.sig(x, deg)
        g = torch.ones_like(s)
        want.append((s.cpu().numpy(), P.sig_backprop(x, s, g, deg).cpu().numpy()))
    L.CUSIG.cusig_amd_set_stream_ordered(1)
    try:
        got = []
        for _ in range(3):
            got = []
            for x, (_, deg) in zip(xs, cases):
                s = P.sig(x, deg)
                got.append((s, P.sig_backprop(x, s, torch.ones_like(s), deg)))
        torch.cuda.synchronize()
    finally:
        L.CUSIG.cusig_amd_set_stream_ordered(0)
    for (s, gr), (ws, wg) in zip(got, want):
        np.testing.assert_allclose(s.cpu().numpy(), ws, rtol=0, atol=0)
        np.testing.assert_allclose(gr.cpu().numpy(), wg, rtol=1e-12, atol=1e-13)


def _alloc_hooks():
    import ctypes
    from pysiglib_amd import _loader as L
    L.CUSIG.cusig_amd_set_alloc_limit.argtypes = (ctypes.c_uint64,)
    L.CUSIG.cusig_amd_set_alloc_limit.restype = None
    L.CUSIG.cusig_amd_alloc_retries.argtypes = ()
    L.CUSIG.cusig_amd_alloc_retries.restype = ctypes.c_int
    return L


def test_out_of_memory_halves_the_batch(P, oracle):
    """A workspace the device cannot hold (forced from the host: requests above a limit fail) makes the call retry on
    halves of its batch, like the reference (siglib/cusig/cu_runtime_utils.h:103-105,212-235); the results are those
    of the undisturbed call, and only a single path that does not fit is an error (a device error, status 100002)."""
    L = _alloc_hooks()
    rng = np.random.default_rng(77)
    b, length, d, deg = 64, 50, 6, 4
    x = np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.3
    ref = oracle.signature(x, deg, n_jobs=-1, time_aug=True)
    g = rng.standard_normal(ref.shape)
    want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1, time_aug=True)
    inc_bytes = b * (length + 1) * (d + 1) * 8      # increments of the augmented path: [b][L + 2][d + 1]
    try:
        L.CUSIG.cusig_shutdown()                     # grown workspaces would hide the limit
        before = L.CUSIG.cusig_amd_alloc_retries()
        L.CUSIG.cusig_amd_set_alloc_limit(inc_bytes // 3)
        fwd = P.sig(dev(x), deg, time_aug=True).cpu().numpy()
        mid = L.CUSIG.cusig_amd_alloc_retries()
        assert mid >= before + 3, (before, mid)      # 64 -> 32 + 32 -> 16 + 16 + 16 + 16
        assert L.CUSIG.cusig_amd_last_sig_nonfinite() == 0
        L.CUSIG.cusig_shutdown()
        bwd = P.sig_backprop(dev(x), dev(ref), dev(g), deg, time_aug=True).cpu().numpy()
        assert L.CUSIG.cusig_amd_alloc_retries() >= mid + 3
        L.CUSIG.cusig_shutdown()
        L.CUSIG.cusig_amd_set_alloc_limit(64)        # not even one path fits
        with pytest.raises(Exception, match="single batch item"):
            P.sig(dev(x), deg, time_aug=True)
    finally:
        L.CUSIG.cusig_amd_set_alloc_limit(0)
    assert level_rel_err(fwd, ref, d + 1, deg) <= 1e-10
    assert bwd_rel_err(bwd, want) <= 1e-10
    np.testing.assert_array_equal(fwd, P.sig(dev(x), deg, time_aug=True).cpu().numpy())


def test_degree_three_matrix_form_falls_back_to_the_sweeps(P, oracle):
    """When the device cannot hold the rows buffer of the degree-3 matrix form, the sweeps serve the call."""
    import ctypes
    L = _alloc_hooks()
    L.CUSIG.cusig_amd_force_degree3.argtypes = (ctypes.c_int,)
    L.CUSIG.cusig_amd_force_degree3.restype = None
    rng = np.random.default_rng(78)
    b, length, d = 8, 40, 20
    x = np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.2
    ref = oracle.signature(x, 3, n_jobs=-1)
    g = rng.standard_normal(ref.shape)
    want = oracle.sig_backprop(x, ref, g, 3, n_jobs=-1)
    rows_bytes = b * (length - 1) * d * d * 8
    try:
        L.CUSIG.cusig_shutdown()
        L.CUSIG.cusig_amd_force_degree3(1)
        L.CUSIG.cusig_amd_set_profiling(1)
        L.CUSIG.cusig_amd_set_alloc_limit(rows_bytes // 2)      # the increments (d instead of d^2 per step) still fit
        fwd = P.sig(dev(x), 3).cpu().numpy()
        assert "degree3" not in L.CUSIG.cusig_amd_last_kernel_name().decode()
        bwd = P.sig_backprop(dev(x), dev(ref), dev(g), 3).cpu().numpy()
        assert "degree3" not in L.CUSIG.cusig_amd_last_kernel_name().decode()
        L.CUSIG.cusig_amd_set_alloc_limit(0)
        P.sig_backprop(dev(x), dev(ref), dev(g), 3)
        assert "degree3" in L.CUSIG.cusig_amd_last_kernel_name().decode()
    finally:
        L.CUSIG.cusig_amd_set_alloc_limit(0)
        L.CUSIG.cusig_amd_force_degree3(-1)
        L.CUSIG.cusig_amd_set_profiling(0)
    assert level_rel_err(fwd, ref, d, 3) <= 1e-10
    assert bwd_rel_err(bwd, want) <= 1e-10


@pytest.mark.parametrize("shape", [(2, 5, 2, 17), (1, 4, 2, 18), (1, 4, 3, 17)])
@pytest.mark.parametrize("scalar_term", [False, True])
def test_degrees_beyond_sixteen_at_their_own_dispatch(P, oracle, shape, scalar_term):
    """Degrees 17 and 18 reach the run-time-degree sweeps without any hook: forward and backward against the oracle
    (262 143 / 524 287 coefficients with two channels, 193 710 244 with three)."""
    b, length, d, deg = shape
    rng = np.random.default_rng(1000 * deg + d)
    x = np.cumsum(rng.standard_normal((b, length, d)), axis=1) * 0.5
    ref = oracle.signature(x, deg, n_jobs=-1, scalar_term=scalar_term)
    g = rng.standard_normal(ref.shape)
    want = oracle.sig_backprop(x, ref, g, deg, n_jobs=-1)
    fwd = P.sig(dev(x), deg, scalar_term=scalar_term)
    got = P.sig_backprop(dev(x), fwd, dev(g), deg).cpu().numpy()
    off = 1 if scalar_term else 0
    assert level_rel_err(fwd.cpu().numpy()[:, off:], ref[:, off:], d, deg) <= 1e-10, shape
    assert bwd_rel_err(got, want) <= 1e-10, shape
