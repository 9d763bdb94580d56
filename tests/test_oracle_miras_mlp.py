"""Pins the CPU oracle of the MIRAS MLP memories MONETA (l_p error, L_q / L2 retention) and YAAD (Huber error,
local + global L2 retention) — core/kernels/moneta_{forward,backward}.cu — without the reference: an independent
numpy forward (matrix products, numpy's own L_q norm), hand-checkable special cases, and finite differences of
the float64 forward with the SiLU slopes of the inner gradient frozen (the reference's backward has no second
derivative of the activation) for every gradient and every error function.  CPU only."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import np_rules as npr

silu = lambda x: x / (1 + np.exp(-x))


def silu_p(x):
    sg = 1 / (1 + np.exp(-x))
    return sg + x * sg * (1 - sg)


def g_fn(e, mode, p1, p2):
    if mode == 1:
        return np.where(np.abs(e) < p1, e, p1 * np.sign(e))
    if abs(p1 - 2) < 1e-6:
        return 2 * e
    if abs(p1 - 1) < 1e-6:
        return np.tanh(p2 * e)
    return p1 * np.tanh(p2 * e) * (e * e + 1e-6) ** ((p1 - 1) / 2)


def np_forward(mode, k, v, q, alpha, theta, w1, w2, p1, p2, lam2, lq_q=2.0, boundary=None, record=None):
    a1, a2 = w1.copy(), w2.copy()
    ys = []
    for t in range(k.shape[0]):
        pre = w1 @ k[t]
        h = silu(pre)
        g = g_fn(w2 @ h - v[t], mode, p1, p2)
        if record is not None:
            record.append(silu_p(pre))
        gpre = (w2.T @ g) * silu_p(pre)
        r1, r2 = 2 * lam2 * w1, 2 * lam2 * w2
        if mode == 1:
            r1 = r1 + 2 * p2 * (w1 - boundary[0])
            r2 = r2 + 2 * p2 * (w2 - boundary[1])
        if mode == 0 and abs(lq_q - 2) >= 1e-6:
            a1 = alpha[t] * a1 - theta[t] * (np.outer(gpre, k[t]) + r1)
            a2 = alpha[t] * a2 - theta[t] * (np.outer(g, h) + r2)
            w1 = a1 * np.linalg.norm(a1.ravel(), ord=lq_q) ** (-(lq_q - 2))
            w2 = a2 * np.linalg.norm(a2.ravel(), ord=lq_q) ** (-(lq_q - 2))
        else:
            w1 = alpha[t] * w1 - theta[t] * (np.outer(gpre, k[t]) + r1)
            w2 = alpha[t] * w2 - theta[t] * (np.outer(g, h) + r2)
        ys.append(w2 @ silu(w1 @ q[t]))
    return np.array(ys), w1, w2


def _inputs(s, d, dh, seed):
    r = np.random.default_rng(seed)
    k, v, q, dy = (r.standard_normal((s, d)) for _ in range(4))
    sig = lambda x: 1 / (1 + np.exp(-x))
    alpha, theta = 0.8 + 0.19 * sig(r.standard_normal(s)), 0.2 * sig(r.standard_normal(s))
    w1, w2 = 0.5 * r.standard_normal((dh, d)), 0.5 * r.standard_normal((d, dh))
    bnd = (w1 + 0.1 * r.standard_normal((dh, d)), w2 + 0.1 * r.standard_normal((d, dh)))
    return k, v, q, alpha, theta, w1, w2, bnd, dy


CASES = [(0, 2.0, 10.0, 2.0), (0, 1.0, 10.0, 2.0), (0, 1.5, 10.0, 2.0), (0, 2.0, 10.0, 3.0), (0, 1.5, 5.0, 4.0),
         (1, 0.7, 0.05, 2.0)]


@pytest.mark.parametrize("mode,p1,p2,lq", CASES)
def test_forward_matches_independent_numpy(mode, p1, p2, lq):
    s, d, dh = 6, 4, 7
    k, v, q, alpha, theta, w1, w2, bnd, _ = _inputs(s, d, dh, 3 + int(10 * p1))
    b = bnd if mode == 1 else None
    y, w1s, w2s = orc.miras_mlp_forward(mode, k, v, q, alpha, theta, w1, w2, dh, p1, p2, 0.01, lq, b)
    yn, w1n, w2n = np_forward(mode, k, v, q, alpha, theta, w1, w2, p1, p2, 0.01, lq, b)
    assert np.abs(y - yn).max() < 1e-11 and np.abs(w1s[-1] - w1n).max() < 1e-11 and np.abs(w2s[-1] - w2n).max() < 1e-11
    assert np.array_equal(w1s[0], w1) and np.array_equal(w2s[0], w2)
    if mode == 1:   # the Huber branch must be exercised on both sides of delta
        e = [w2s[t] @ silu(w1s[t] @ k[t]) - v[t] for t in range(s)]
        assert (np.abs(e) < p1).any() and (np.abs(e) > p1).any()


def test_theta_zero_only_decays_and_lq_keeps_the_direction():
    s, d, dh = 4, 3, 5
    k, v, q, alpha, theta, w1, w2, _, _ = _inputs(s, d, dh, 9)
    _, w1s, w2s = orc.miras_mlp_forward(0, k, v, q, alpha, np.zeros(s), w1, w2, dh, 2.0, 10.0, 0.3)
    assert np.allclose(w1s[-1], np.prod(alpha) * w1, atol=1e-14) and np.allclose(w2s[-1], np.prod(alpha) * w2, atol=1e-14)
    _, w1q, _ = orc.miras_mlp_forward(0, k, v, q, alpha, np.zeros(s), w1, w2, dh, 2.0, 10.0, 0.3, lq_q=3.0)
    cos = (w1q[-1] * w1).sum() / np.linalg.norm(w1q[-1]) / np.linalg.norm(w1)
    assert abs(cos - 1) < 1e-12 and not np.allclose(w1q[-1], w1s[-1])


@pytest.mark.parametrize("mode,p1,p2", [(0, 2.0, 10.0), (0, 1.0, 3.0), (0, 1.5, 3.0), (1, 0.7, 0.05)])
def test_backward_matches_finite_differences_with_frozen_silu_slopes(mode, p1, p2):
    s, d, dh = 5, 3, 4
    k, v, q, alpha, theta, w1, w2, bnd, dy = _inputs(s, d, dh, 21 + int(10 * p1))
    b = bnd if mode == 1 else None
    rec = []
    np_forward(mode, k, v, q, alpha, theta, w1, w2, p1, p2, 0.02, 2.0, b, record=rec)
    fix = np.array(rec)
    y0, w1s, w2s = orc.miras_mlp_forward(mode, k, v, q, alpha, theta, w1, w2, dh, p1, p2, 0.02, 2.0, b)
    P = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, w1=w1, w2=w2)

    def loss():
        y, _, _ = orc.miras_mlp_forward(mode, k, v, q, alpha, theta, w1, w2, dh, p1, p2, 0.02, 2.0, b, slope_fix=fix)
        return float((y * dy).sum())

    assert abs(loss() - float((y0 * dy).sum())) < 1e-12
    fd = npr.fd_grads(loss, P)
    r = np.random.default_rng(1)
    k0, v0 = r.standard_normal((s, d)), r.standard_normal((s, d))   # d_k is added to, d_v subtracted from
    g = orc.miras_mlp_backward(mode, k, v, q, alpha, theta, w1s, w2s, dy, dh, p1, p2, 0.02, b, d_k0=k0, d_v0=v0)
    an = dict(k=g["d_k"] - k0, v=g["d_v"] - v0, q=g["d_q"], alpha=g["d_alpha"], theta=g["d_theta"], w1=g["d_w1"],
              w2=g["d_w2"])
    for n in P:
        scale = max(np.abs(fd[n]).max(), 1e-3)
        assert np.abs(fd[n] - an[n]).max() / scale < 1e-5, n
