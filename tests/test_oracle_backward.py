"""Pins oracle/backward.py (the CPU statement of the backward library calls) by what the mathematics fixes: adjoint
identities against the forward oracle, a pure-Python brute force for max pooling, finite differences for log-softmax.
A dropped term, a wrong sign, a transposed filter index or an off-by-one in the window arithmetic fails one of them."""
import numpy as np
import pytest

import oracle
from oracle import backward as ob

CONV_CASES = [
    # n, c, h, w, f, k, stride, pad, dilation, groups
    (2, 6, 9, 8, 4, 3, 2, 1, 1, 2),
    (1, 4, 7, 7, 8, 3, 1, 1, 2, 1),
    (2, 8, 6, 6, 8, 1, 1, 0, 1, 4),
    (1, 3, 10, 11, 5, 5, 3, 2, 1, 1),
]


@pytest.mark.parametrize("case", CONV_CASES)
def test_convolution_gradients_are_the_adjoints_of_the_forward_oracle(case):
    n, c, h, w_, f, k, s, p, d, g = case
    rng = np.random.default_rng(sum(case))
    x = rng.standard_normal((n, c, h, w_)).astype(np.float32)
    w = rng.standard_normal((f, c // g, k, k)).astype(np.float32)
    y = oracle.conv2d_nchw(x, w, (s, s), (p, p), (d, d), g).astype(np.float64)
    dy = rng.standard_normal(y.shape)
    dx = ob.conv2d_backward_data(w, dy, x.shape, (s, s), (p, p), (d, d), g)
    dw = ob.conv2d_backward_filter(x, dy, w.shape, (s, s), (p, p), (d, d), g)
    lhs = (y * dy).sum()
    scale = (np.abs(y) * np.abs(dy)).sum()
    assert abs(lhs - (x.astype(np.float64) * dx).sum()) <= 1e-5 * scale
    assert abs(lhs - (w.astype(np.float64) * dw).sum()) <= 1e-5 * scale
    # the identity holds for every dy, so it pins every coefficient: check single-element probes too
    probe = np.zeros_like(dy)
    probe[0, f - 1, y.shape[2] // 2, y.shape[3] - 1] = 1.0
    dxp = ob.conv2d_backward_data(w, probe, x.shape, (s, s), (p, p), (d, d), g)
    assert abs(y[0, f - 1, y.shape[2] // 2, y.shape[3] - 1] - (x.astype(np.float64) * dxp).sum()) <= 1e-5 * scale


def brute_force_max_pool_backward(x, dy, k, s, p):
    n, c, ih, iw = x.shape
    dx = np.zeros(x.shape, np.float64)
    for ni in range(n):
        for ci in range(c):
            for oy in range(dy.shape[2]):
                for ox in range(dy.shape[3]):
                    best, where = None, None
                    for ry in range(k):
                        for rx in range(k):
                            yy, xx = oy * s - p + ry, ox * s - p + rx
                            if 0 <= yy < ih and 0 <= xx < iw and (best is None or x[ni, ci, yy, xx] > best):
                                best, where = x[ni, ci, yy, xx], (yy, xx)
                    dx[ni, ci, where[0], where[1]] += dy[ni, ci, oy, ox]
    return dx


@pytest.mark.parametrize("k,s,p", [(3, 2, 1), (2, 2, 0), (3, 1, 1)])
def test_max_pool_gradient_goes_to_the_first_maximum(k, s, p):
    rng = np.random.default_rng(k * 10 + s)
    # few distinct values: ties inside windows are common, so the tie rule is exercised
    x = rng.integers(0, 4, (2, 3, 7, 8)).astype(np.float32)
    oh = (7 + 2 * p - k) // s + 1
    ow = (8 + 2 * p - k) // s + 1
    dy = rng.standard_normal((2, 3, oh, ow))
    got = ob.pool2d_backward(x, dy, (k, k), (s, s), (p, p), "max")
    np.testing.assert_allclose(got, brute_force_max_pool_backward(x, dy, k, s, p), rtol=0, atol=1e-12)
    assert abs(got.sum() - dy.sum()) < 1e-9


@pytest.mark.parametrize("exclusive", [True, False])
def test_average_pool_gradient_is_the_adjoint_of_the_forward_oracle(exclusive):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 9, 10)).astype(np.float32)
    y = oracle.pool2d_nchw(x, (3, 3), (2, 2), (1, 1, 1, 1), "avg", exclusive=exclusive).astype(np.float64)
    dy = rng.standard_normal(y.shape)
    dx = ob.pool2d_backward(x, dy, (3, 3), (2, 2), (1, 1), "avg", exclusive=exclusive)
    assert abs((y * dy).sum() - (x.astype(np.float64) * dx).sum()) <= 1e-5 * (np.abs(y) * np.abs(dy)).sum()


def test_log_softmax_gradient_matches_finite_differences():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 7)).astype(np.float64)
    dy = rng.standard_normal((3, 7))

    def log_softmax(v):
        m = v.max(axis=1, keepdims=True)
        return v - m - np.log(np.exp(v - m).sum(axis=1, keepdims=True))

    got = ob.log_softmax_backward(log_softmax(x), dy, axis=1)
    eps = 1e-6
    for i in range(3):
        for j in range(7):
            xp, xm = x.copy(), x.copy()
            xp[i, j] += eps
            xm[i, j] -= eps
            fd = ((log_softmax(xp) - log_softmax(xm)) * dy).sum() / (2 * eps)
            assert abs(got[i, j] - fd) < 1e-6
