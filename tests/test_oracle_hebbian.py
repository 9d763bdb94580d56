"""Pins the CPU oracle of the Hebbian rule (core/src/dispatch.rs:1566-1660) without the reference:
the closed form of the linear recurrence written with numpy cumulative products, hand-checkable special
cases, central finite differences of the double-precision forward for every gradient, and the
checkpoint / segment compositions of core/kernels/hebbian_{forward,backward}.cu.  CPU only."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests import np_rules as npr


def _inputs(s, d, seed, dt=np.float64):
    r = np.random.default_rng(seed)
    k, v, q, dy = (r.standard_normal((s, d)) for _ in range(4))
    alpha = 1 / (1 + np.exp(-r.standard_normal(s)))
    m0 = 0.3 * r.standard_normal((d, d))
    return [np.ascontiguousarray(x, dt) for x in (k, v, q, alpha, m0, dy)]


def _closed_form(k, v, q, alpha, m0):
    """M_t = P_t M_0 + sum_{u<t} (P_t / P_{u+1}) v_u k_u^T with P_t = prod_{u<t} (1 - alpha_u)."""
    s, d = k.shape
    P = np.concatenate([[1.0], np.cumprod(1.0 - alpha)])
    ms = np.empty((s + 1, d, d))
    for t in range(s + 1):
        w = P[t] / P[1:t + 1]
        ms[t] = P[t] * m0 + np.einsum("u,ui,uj->ij", w, v[:t], k[:t])
    y = np.einsum("tij,tj->ti", ms[1:], q)
    return y, ms


def test_forward_is_the_closed_form_of_the_recurrence():
    k, v, q, alpha, m0, _ = _inputs(9, 5, 1)
    alpha = np.clip(alpha, 0.05, 0.9)   # keeps the ratios P_t / P_u well conditioned
    y, ms = orc.hebbian_forward(k, v, q, alpha, m0)
    yc, mc = _closed_form(k, v, q, alpha, m0)
    assert np.abs(ms - mc).max() < 1e-12 and np.abs(y - yc).max() < 1e-12
    y32, ms32 = orc.hebbian_forward(*[x.astype(np.float32) for x in (k, v, q, alpha, m0)])
    assert np.abs(y32 - yc).max() < 2e-5 * max(1.0, np.abs(yc).max())


def test_special_cases():
    k, v, q, alpha, m0, _ = _inputs(6, 4, 2)
    # alpha = 1 forgets everything: M_{t+1} = v_t k_t^T, y_t = v_t (k_t . q_t)
    y, ms = orc.hebbian_forward(k, v, q, np.ones(6), m0)
    assert np.allclose(ms[1:], np.einsum("ti,tj->tij", v, k), atol=1e-14)
    assert np.allclose(y, v * (k * q).sum(1, keepdims=True), atol=1e-13)
    # alpha = 0 is a plain sum of outer products on top of M_0
    y, ms = orc.hebbian_forward(k, v, q, np.zeros(6), m0)
    assert np.allclose(ms[-1], m0 + v.T @ k, atol=1e-13)
    # one token, M_0 = 0, orthonormal key: reading with the key returns the value
    e0 = np.eye(4)[:1]
    y, _ = orc.hebbian_forward(e0, v[:1], e0, np.array([0.3]), np.zeros((4, 4)))
    assert np.allclose(y, v[:1], atol=1e-15)


def test_m_norm_projection_bounds_the_state():
    k, v, q, alpha, m0, _ = _inputs(8, 4, 3)
    _, ms = orc.hebbian_forward(k, v, q, alpha, m0, m_norm_max=0.7)
    assert np.all(np.linalg.norm(ms[1:].reshape(8, -1), axis=1) <= 0.7 * (1 + 1e-12))
    _, free = orc.hebbian_forward(k, v, q, alpha, m0)
    assert np.linalg.norm(free[1:].reshape(8, -1), axis=1).max() > 0.7, "projection must be active"


def test_backward_matches_finite_differences():
    s, d = 7, 4
    k, v, q, alpha, m0, dy = _inputs(s, d, 4)
    P = dict(k=k, v=v, q=q, alpha=alpha, m0=m0)

    def loss():
        y, _ = orc.hebbian_forward(k, v, q, alpha, m0)
        return float((y * dy).sum())

    fd = npr.fd_grads(loss, P)
    _, ms = orc.hebbian_forward(k, v, q, alpha, m0)
    g = orc.hebbian_backward(k, v, q, alpha, ms, dy)
    an = dict(k=g["d_k"], v=g["d_v"], q=g["d_q"], alpha=g["d_alpha"], m0=g["d_m"])
    for n in P:
        scale = max(np.abs(fd[n]).max(), 1e-3)
        assert np.abs(fd[n] - an[n]).max() / scale < 2e-6, n


def test_float_backward_tracks_double_backward():
    k, v, q, alpha, m0, dy = _inputs(20, 8, 5)
    _, ms = orc.hebbian_forward(k, v, q, alpha, m0)
    g64 = orc.hebbian_backward(k, v, q, alpha, ms, dy)
    f = [x.astype(np.float32) for x in (k, v, q, alpha, m0, dy)]
    _, ms32 = orc.hebbian_forward(*f[:5])
    g32 = orc.hebbian_backward(f[0], f[1], f[2], f[3], ms32, f[5])
    for n in g64:
        assert np.abs(g32[n] - g64[n]).max() < 2e-5 * max(1.0, np.abs(g64[n]).max()), n


@pytest.mark.parametrize("C", [1, 4, 5, 64])
def test_checkpoints_and_segments_compose_to_the_full_backward(C):
    s, d = 13, 4
    k, v, q, alpha, m0, dy = _inputs(s, d, 6)
    y, ms = orc.hebbian_forward(k, v, q, alpha, m0)
    yc, ck = orc.hebbian_forward(k, v, q, alpha, m0, checkpoint_interval=C)
    ends = [t + 1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s]
    assert ck.shape[0] == 1 + len(ends) == orc.checkpoint_count(s, C)
    assert np.array_equal(yc, y) and np.array_equal(ck, ms[[0] + ends])
    full = orc.hebbian_backward(k, v, q, alpha, ms, dy)
    # reverse over the segments, each with its own local trajectory replayed from its checkpoint
    seed, got = None, {n: np.zeros_like(full[n]) for n in ("d_k", "d_v", "d_q", "d_alpha")}
    starts = [0] + ends[:-1]
    for i in reversed(range(len(ends))):
        lo, hi = starts[i], ends[i]
        _, local = orc.hebbian_forward(k[lo:hi], v[lo:hi], q[lo:hi], alpha[lo:hi], ck[i])
        pad = lambda x: np.concatenate([np.zeros((lo,) + x.shape[1:]), x])   # range functions index by global t
        g = orc.hebbian_backward(pad(k[lo:hi]), pad(v[lo:hi]), pad(q[lo:hi]), pad(alpha[lo:hi]), local,
                                 pad(dy[lo:hi]), t_lo=lo, t_hi=hi, d_m_seed=seed)
        for n in got:
            got[n][lo:hi] = g[n][lo:hi]
        seed = g["d_m"]
    for n in got:
        assert np.allclose(got[n], full[n], atol=1e-13), n
    assert np.allclose(seed, full["d_m"], atol=1e-13)
