"""Known-answer data for sig_combine / transform_path and their backward passes.

The values are the hand-computed vectors held by the reference's own unit tests
(siglib/cpsig_unit_testing/cp_test_signature.cpp:64-72,409-446 and
siglib/cpsig_unit_testing/cp_test_misc.cpp:364-503); they are data, shared by the oracle tests and the GPU tests.
"""
import numpy as np

# (sig1, sig2, expected, dimension, degree), scalar term included
COMBINE = [
    ([1., 1., 1., .5, .5, .5, .5], [1., 1., 1., .5, .5, .5, .5], [1., 2., 2., 2., 2., 2., 2.], 2, 2),
]

# (derivs, sig1, sig2, expected d1, expected d2, dimension, degree), scalar term included
COMBINE_BACKPROP = [
    ([1., 1., 2., 3., 4., 5., 6.], [1., 1., 1., .5, .5, .5, .5], [1., 0., 1., 0., 1., -1., .5],
     [0., 5., 8., 3., 4., 5., 6.], [0., 9., 12., 3., 4., 5., 6.], 2, 2),
    ([1., 1., 2., 3., 4., 5., 6.], [1., 0., 1., 0., 1., -1., .5], [1., 1., 1., .5, .5, .5, .5],
     [0., 8., 13., 3., 4., 5., 6.], [0., 6., 8., 3., 4., 5., 6.], 2, 2),
]

# (path (len, dim), kwargs, expected)
TRANSFORM = [
    ([[0., 0.], [1., 2.], [3., 4.]], dict(time_aug=True), [[0., 0., 0.], [1., 2., .5], [3., 4., 1.]]),
    ([[0., 0.], [1., 2.], [3., 4.]], dict(time_aug=True, end_time=2.), [[0., 0., 0.], [1., 2., 1.], [3., 4., 2.]]),
    ([[1., 2.], [3., 4.], [5., 6.]], dict(lead_lag=True),
     [[1., 2., 1., 2.], [1., 2., 3., 4.], [3., 4., 3., 4.], [3., 4., 5., 6.], [5., 6., 5., 6.]]),
    ([[1., 2.], [3., 4.], [5., 6.]], dict(time_aug=True, lead_lag=True),
     [[1., 2., 1., 2., 0.], [1., 2., 3., 4., .25], [3., 4., 3., 4., .5], [3., 4., 5., 6., .75], [5., 6., 5., 6., 1.]]),
]


def _iota(*shape):
    return np.arange(int(np.prod(shape)), dtype=np.float64).reshape(shape)


def _lead_lag_ones(length, dim):
    out = np.full((length, dim), 4.)
    out[0] = 3.
    out[-1] = 3.
    return out


# (derivs (transformed len, transformed dim), kwargs, expected (len, dim))
TRANSFORM_BACKPROP = [
    (np.ones((3, 3)), dict(time_aug=True), np.ones((3, 2))),
    (_iota(5, 4), dict(lead_lag=True), np.array([[6., 9.], [36., 40.], [48., 51.]])),
    (np.ones((199, 10)), dict(lead_lag=True), _lead_lag_ones(100, 5)),
    (np.ones((5, 5)), dict(time_aug=True, lead_lag=True), np.array([[3., 3.], [4., 4.], [3., 3.]])),
]
