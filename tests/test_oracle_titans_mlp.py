"""Pins the CPU oracle of the Titans rule with an MLP memory (core/kernels/titans_mlp_{forward,backward}.cu)
without the reference: an independent numpy forward written with matrix operations, the linear special case
that reduces to the matrix-memory Titans rule, and finite differences of the double-precision forward for
every gradient.  The reference's backward treats act'(pre) in the inner gradient as a constant (no second
derivative of the activation), so the differences are taken on a forward whose act' factors are frozen at the
recorded values; for ReLU the second derivative vanishes and the plain forward is differenced too.  CPU only."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import np_rules as npr

C0, A0 = 0.7978845608028654, 0.044715


def _act(x, act):
    if act == 0:
        return 0.5 * x * (1 + np.tanh(C0 * (x + A0 * x ** 3)))
    if act == 1:
        return x / (1 + np.exp(-x))
    return np.maximum(x, 0)


def _act_prime(x, act):
    if act == 0:
        t = np.tanh(C0 * (x + A0 * x ** 3))
        return 0.5 * (1 + t) + 0.5 * x * (1 - t * t) * C0 * (1 + 3 * A0 * x * x)
    if act == 1:
        sg = 1 / (1 + np.exp(-x))
        return sg + x * sg * (1 - sg)
    return (x > 0).astype(x.dtype)


def _unpack(m, d, dh):
    w1 = m[:dh * d].reshape(dh, d)
    b1 = m[dh * d:dh * d + dh]
    w2 = m[dh * d + dh:2 * dh * d + dh].reshape(d, dh)
    return w1, b1, w2, m[2 * dh * d + dh:]


def np_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act, m_norm_max=0.0, actp_fix=None, record=None):
    """Independent restatement with matrix products; record: list that receives act'(pre) per token."""
    s, d = k.shape
    m, mom = m0.copy(), s0.copy()
    ys = []
    for t in range(s):
        w1, b1, w2, b2 = _unpack(m, d, dh)
        pre = w1 @ k[t] + b1
        h = _act(pre, act)
        e = w2 @ h + b2 - v[t]
        ap = _act_prime(pre, act) if actp_fix is None else actp_fix[t]
        if record is not None:
            record.append(_act_prime(pre, act))
        gpre = (w2.T @ e) * ap
        grad = np.concatenate([np.outer(gpre, k[t]).ravel(), gpre, np.outer(e, h).ravel(), e])
        mom = eta[t] * mom - theta[t] * grad
        m = (1 - alpha[t]) * m + mom
        if m_norm_max > 0 and np.linalg.norm(m) > m_norm_max:
            m = m * (m_norm_max / np.linalg.norm(m))
        w1, b1, w2, b2 = _unpack(m, d, dh)
        ys.append(w2 @ _act(w1 @ q[t] + b1, act) + b2)
    return np.array(ys), m, mom


def _inputs(s, d, dh, seed):
    r = np.random.default_rng(seed)
    k, v, q, dy = (r.standard_normal((s, d)) for _ in range(4))
    k /= np.linalg.norm(k, axis=1, keepdims=True)
    sig = lambda x: 1 / (1 + np.exp(-x))
    alpha, theta, eta = 0.2 * sig(r.standard_normal(s)), 0.3 * sig(r.standard_normal(s)), sig(r.standard_normal(s))
    n = orc.mlp_state_size(d, dh)
    m0, s0 = 0.4 * r.standard_normal(n), 0.05 * r.standard_normal(n)
    return k, v, q, alpha, theta, eta, m0, s0, dy


@pytest.mark.parametrize("act", [0, 1, 2])
def test_forward_matches_independent_numpy(act):
    s, d, dh = 7, 5, 9   # d_hidden neither a power of two nor a multiple of d
    k, v, q, alpha, theta, eta, m0, s0, _ = _inputs(s, d, dh, 10 + act)
    y, ms, ss = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act)
    yn, mn, sn = np_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act)
    assert np.abs(y - yn).max() < 1e-12 and np.abs(ms[-1] - mn).max() < 1e-12 and np.abs(ss[-1] - sn).max() < 1e-12
    assert np.array_equal(ms[0], m0) and np.array_equal(ss[0], s0)
    y32, _, _ = orc.titans_mlp_forward(*[x.astype(np.float32) for x in (k, v, q, alpha, theta, eta, m0, s0)], dh, act)
    assert np.abs(y32 - yn).max() < 3e-5 * max(1.0, np.abs(yn).max())


def test_projection_bounds_the_state_and_is_a_noop_when_large():
    s, d, dh = 6, 4, 6
    k, v, q, alpha, theta, eta, m0, s0, _ = _inputs(s, d, dh, 20)
    free = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 0)
    cap = 0.8 * np.linalg.norm(free[1][1:], axis=1).max()
    y, ms, _ = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 0, m_norm_max=cap)
    assert np.all(np.linalg.norm(ms[1:], axis=1) <= cap * (1 + 1e-12))
    yn, _, _ = np_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 0, m_norm_max=cap)
    assert np.abs(y - yn).max() < 1e-12
    big = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 0, m_norm_max=1e6)
    assert np.array_equal(big[0], free[0])


def test_with_relu_wide_open_the_memory_is_a_product_of_two_matrices():
    """ReLU with all pre-activations positive and zero biases kept out of the update is linear: y = W2 W1 q."""
    s, d, dh = 3, 3, 4
    r = np.random.default_rng(5)
    w1, w2 = np.abs(r.standard_normal((dh, d))) + 0.5, r.standard_normal((d, dh))
    k = np.abs(r.standard_normal((s, d))) + 0.1
    q = np.abs(r.standard_normal((s, d))) + 0.1
    v = r.standard_normal((s, d))
    m0 = np.concatenate([w1.ravel(), np.zeros(dh), w2.ravel(), np.zeros(d)])
    zero = np.zeros(s)
    y, ms, _ = orc.titans_mlp_forward(k, v, q, zero, zero, zero, m0, np.zeros_like(m0), dh, 2)   # theta = 0: no update
    assert np.allclose(y, q @ (w2 @ w1).T, atol=1e-13) and np.array_equal(ms[-1], m0)


@pytest.mark.parametrize("act", [0, 1, 2])
def test_backward_matches_finite_differences_with_frozen_activation_slopes(act):
    s, d, dh = 5, 3, 4
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, dh, 30 + act)
    rec = []
    np_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act, record=rec)
    fix = np.array(rec)
    yf, _, _ = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act, actp_fix=fix)
    y0, ms, ss = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act)
    assert np.abs(yf - y0).max() < 1e-13, "freezing at the recorded values changes nothing at the base point"
    P = dict(k=k, v=v, q=q, alpha=alpha, theta=theta, eta=eta, m0=m0, s0=s0)

    def loss():
        y, _, _ = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, act, actp_fix=fix)
        return float((y * dy).sum())

    fd = npr.fd_grads(loss, P)
    g = orc.titans_mlp_backward(k, v, q, alpha, theta, eta, ms, ss, dy, dh, act)
    an = dict(k=g["d_k"], v=g["d_v"], q=g["d_q"], alpha=g["d_alpha"], theta=g["d_theta"], eta=g["d_eta"],
              m0=g["d_m"], s0=g["d_s"])
    for n in P:
        scale = max(np.abs(fd[n]).max(), 1e-3)
        assert np.abs(fd[n] - an[n]).max() / scale < 5e-6, n


def test_relu_backward_is_the_exact_gradient():
    """act'' = 0 for ReLU away from the kinks: the analytic backward must match the plain forward's differences."""
    s, d, dh = 4, 3, 4
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, dh, 41)
    y0, ms, ss = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 2)
    P = dict(k=k, v=v, q=q, m0=m0)

    def loss():
        y, _, _ = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 2)
        return float((y * dy).sum())

    fd = npr.fd_grads(loss, P)
    g = orc.titans_mlp_backward(k, v, q, alpha, theta, eta, ms, ss, dy, dh, 2)
    for n, a in (("k", g["d_k"]), ("v", g["d_v"]), ("q", g["d_q"]), ("m0", g["d_m"])):
        scale = max(np.abs(fd[n]).max(), 1e-3)
        assert np.abs(fd[n] - a).max() / scale < 5e-6, n


def test_float_backward_tracks_double_backward():
    s, d, dh = 12, 8, 16
    k, v, q, alpha, theta, eta, m0, s0, dy = _inputs(s, d, dh, 50)
    _, ms, ss = orc.titans_mlp_forward(k, v, q, alpha, theta, eta, m0, s0, dh, 0)
    g64 = orc.titans_mlp_backward(k, v, q, alpha, theta, eta, ms, ss, dy, dh, 0)
    f = [x.astype(np.float32) for x in (k, v, q, alpha, theta, eta, m0, s0, dy)]
    _, ms32, ss32 = orc.titans_mlp_forward(*f[:8], dh, 0)
    g32 = orc.titans_mlp_backward(*f[:6], ms32, ss32, f[8], dh, 0)
    for n in g64:
        assert np.abs(g32[n] - g64[n]).max() < 5e-5 * max(1.0, np.abs(g64[n]).max()), n
