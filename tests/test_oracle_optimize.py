"""Pins of the oracle's optimizer functions by what the mathematics fixes: closed forms of the
momentum / Nesterov / l2 / running-average recurrences and the round trip of the flat copies."""
import numpy as np
import pytest

import oracle


def test_add_scaled_and_online_closed_forms():
    rng = np.random.default_rng(0)
    x = rng.standard_normal(1000).astype(np.float32)
    y0 = rng.standard_normal(1000).astype(np.float32)
    y = y0.copy()
    oracle.array_add_scaled(0.25, x, -1.5, y)
    np.testing.assert_allclose(y, 0.25 * x.astype(np.float64) - 1.5 * y0.astype(np.float64), rtol=0, atol=3e-7)
    # online average: after t updates toward a constant x, y_t = x + (1-a)^t (y_0 - x)
    y = y0.copy()
    a = 0.125
    for _ in range(7):
        oracle.array_add_online(a, x, y)
    want = x.astype(np.float64) + (1 - a) ** 7 * (y0.astype(np.float64) - x)
    np.testing.assert_allclose(y, want, rtol=0, atol=1e-6)
    # a == 1 lands on x up to one rounding of the difference
    y = y0.copy()
    oracle.array_add_online(1.0, x, y)
    np.testing.assert_allclose(y, x, rtol=0, atol=2.5e-7)


def test_flat_store_load_round_trip_and_offsets():
    rng = np.random.default_rng(1)
    arrays = [rng.standard_normal(s).astype(np.float32) for s in [(3, 4), (1,), (0,), (5, 2, 2), (7,)]]
    dim = oracle.flat_store(arrays, None, 0)
    assert dim == 12 + 1 + 0 + 20 + 7
    flat = np.full(dim + 5, -7.0, np.float32)
    end = oracle.flat_store(arrays, flat, 3)
    assert end == dim + 3
    assert (flat[:3] == -7).all() and (flat[end:] == -7).all()
    np.testing.assert_array_equal(flat[3:15], arrays[0].ravel())
    np.testing.assert_array_equal(flat[15:16], arrays[1].ravel())
    np.testing.assert_array_equal(flat[16:36], arrays[3].ravel())
    np.testing.assert_array_equal(flat[36:43], arrays[4].ravel())
    back = [np.zeros_like(a) for a in arrays]
    assert oracle.flat_load(back, flat, 3) == end
    for a, b in zip(arrays, back):
        np.testing.assert_array_equal(a, b)


def _run(steps, grads_fn, p0, l2, mu, alphas, nesterov):
    n = p0.size
    p = p0.copy()
    m = np.zeros(n, np.float32)
    lag = np.zeros(n, np.float32)
    sg = np.zeros(n, np.float32)
    hist = []
    for t in range(steps):
        oracle.sgd_step(grads_fn(t, p), p, m, lag, sg, l2, mu, alphas[t], alphas[t + 1], nesterov)
        hist.append((p.copy(), m.copy(), lag.copy(), sg.copy()))
    return hist


def test_sgd_momentum_closed_form_constant_gradient():
    # constant gradient g split over 3 ranks: m_t = g (1-mu^t)/(1-mu), p_t = p_0 - alpha * sum_{s<=t} m_s
    rng = np.random.default_rng(2)
    n = 257
    parts = [rng.standard_normal(n).astype(np.float32) for _ in range(3)]
    g = sum(x.astype(np.float64) for x in parts)
    p0 = rng.standard_normal(n).astype(np.float32)
    mu, alpha, T = 0.9, 0.05, 12
    hist = _run(T, lambda t, p: parts, p0, 0.0, mu, [alpha] * (T + 1), False)
    msum = np.zeros(n)
    for t in range(1, T + 1):
        m_t = g * (1 - mu ** t) / (1 - mu)
        msum += m_t
        p, m, lag, sg = hist[t - 1]
        np.testing.assert_allclose(sg, g, rtol=0, atol=1e-6)
        np.testing.assert_allclose(m, m_t, rtol=2e-6, atol=1e-6)
        np.testing.assert_allclose(p, p0 - alpha * msum, rtol=0, atol=2e-5)
        np.testing.assert_array_equal(lag, p)  # without Nesterov the lagged copy is the new parameter


def test_sgd_l2_shrinks_parameters_geometrically():
    # zero gradient, no momentum: p_t = (1 - alpha*l2)^t p_0
    rng = np.random.default_rng(3)
    p0 = rng.standard_normal(300).astype(np.float32)
    z = np.zeros(300, np.float32)
    alpha, l2, T = 0.1, 0.5, 9
    hist = _run(T, lambda t, p: [z, z], p0, l2, 0.0, [alpha] * (T + 1), False)
    np.testing.assert_allclose(hist[-1][0], (1 - alpha * l2) ** T * p0.astype(np.float64), rtol=1e-5, atol=1e-7)
    # the regularised gradient that comes back is l2 * (parameter before the step)
    np.testing.assert_allclose(hist[0][3], l2 * p0, rtol=1e-6, atol=0)


def test_sgd_nesterov_matches_textbook_lookahead():
    # Textbook (Sutskever) Nesterov momentum with a constant step:
    #   v_{t+1} = mu v_t - alpha grad(theta_t + mu v_t);  theta_{t+1} = theta_t + v_{t+1}
    # The optimizer keeps the look-ahead point theta + mu v as `param` (where the next gradient is taken)
    # and the plain iterate theta as `lagged`.  Run the textbook form in float64 on f(p) = 0.5 |p|^2.
    rng = np.random.default_rng(4)
    n = 64
    p0 = rng.standard_normal(n).astype(np.float32)
    mu, alpha, T = 0.8, 0.3, 10
    hist = _run(T, lambda t, p: [p.copy()], p0, 0.0, mu, [alpha] * (T + 1), True)
    theta = p0.astype(np.float64)
    v = np.zeros(n)
    for t in range(T):
        v = mu * v - alpha * (theta + mu * v)
        theta = theta + v
        np.testing.assert_allclose(hist[t][2], theta, rtol=0, atol=2e-6)          # lagged = iterate
        np.testing.assert_allclose(hist[t][0], theta + mu * v, rtol=0, atol=2e-6)  # param = look-ahead point
        np.testing.assert_allclose(hist[t][1], -v / alpha, rtol=0, atol=1e-5)      # momentum_grad = -v/alpha
    assert np.abs(hist[-1][2]).max() < 0.1 * np.abs(p0).max()  # and it contracts on the quadratic
    # a changing step: this step's size multiplies the gradient, the NEXT step's size the momentum term
    # (include/arraydiff/optimize.hh:488-492)
    alphas = [0.3 / (1 + 0.2 * t) for t in range(T + 1)]
    hist = _run(T, lambda t, p: [p.copy()], p0, 0.0, mu, alphas, True)
    p = p0.astype(np.float64)
    m = np.zeros(n)
    for t in range(T):
        g = p.copy()
        m = g + mu * m
        lag = p - alphas[t] * g
        p = lag - alphas[t + 1] * mu * m
        np.testing.assert_allclose(hist[t][2], lag, rtol=0, atol=2e-6)
        np.testing.assert_allclose(hist[t][0], p, rtol=0, atol=2e-6)
    # mu == 0: Nesterov and plain SGD coincide
    a = _run(3, lambda t, p: [p.copy()], p0, 0.0, 0.0, alphas, True)
    b = _run(3, lambda t, p: [p.copy()], p0, 0.0, 0.0, alphas, False)
    np.testing.assert_array_equal(a[-1][0], b[-1][0])


def test_stat_step_copies_running_average():
    rng = np.random.default_rng(5)
    avg = rng.standard_normal(100).astype(np.float32)
    run = rng.standard_normal(100).astype(np.float32)
    run0 = run.copy()
    stat = np.zeros(100, np.float32)
    oracle.stat_step(0.003, avg, run, stat)
    np.testing.assert_array_equal(stat, run)
    np.testing.assert_allclose(run, run0 + 0.003 * (avg.astype(np.float64) - run0), rtol=0, atol=2e-7)
