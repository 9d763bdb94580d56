"""GPU parity of the Titans rule with an MLP memory through the C ABI against the CPU oracle: the reference's
own recipes (core/tests/test_titans_mlp_cuda.rs: d = 8, expansion 4, rand_buf seeds 42-45, ramped gates,
absolute 1e-4) for the three activations, with the norm projection active, longer sequences, a non-zero
initial momentum, batches and a hidden size that is not a power of two; backward at relative 1e-4."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_abs, assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
f32 = np.float32
F32_MAX = orc.F32_MAX


def _recipe(seq_len, d, dh, seed0=42, s_seed=None):
    rb = orc.simple_rng_uniform
    n = orc.mlp_state_size(d, dh)
    k, v, q = (rb(seq_len * d, seed0 + i).reshape(seq_len, d) for i in range(3))
    t = np.arange(seq_len, dtype=f32)
    alpha, theta, eta = (0.05 + 0.02 * t).astype(f32), (0.01 + 0.005 * t).astype(f32), (0.9 - 0.05 * t).astype(f32)
    m0 = rb(n, seed0 + 3)
    s0 = np.zeros(n, f32) if s_seed is None else rb(n, s_seed)
    return k, v, q, alpha, theta, np.clip(eta, 0.05, None), m0, s0


def gpu_forward(x, dh, act, m_norm_max):
    """x: list of per-chain recipes"""
    B = len(x)
    s, d = x[0][0].shape
    n = orc.mlp_state_size(d, dh)
    st = lambda i: dev(np.stack([c[i] for c in x]))
    ms, ss, y = zeros(B, s + 1, n), zeros(B, s + 1, n), zeros(B, s, d)
    D.call("titans_mlp_forward_f32_cuda", st(0), st(1), st(2), st(3), st(4), st(5), st(6), st(7), ms, ss, y,
           s, d, dh, B, s * d, (s + 1) * n, act, m_norm_max)
    torch.cuda.synchronize()
    return host(y), host(ms), host(ss)


@pytest.mark.parametrize("act", [0, 1, 2])
@pytest.mark.parametrize("seq_len,d,dh,m_norm_max,s_seed", [(4, 8, 32, 100.0, None), (1, 8, 32, 100.0, None),
                                                            (4, 8, 32, 1.0, None), (16, 8, 32, F32_MAX, None),
                                                            (4, 8, 32, 100.0, 99), (4, 8, 24, 100.0, None)])
def test_reference_forward_recipes(act, seq_len, d, dh, m_norm_max, s_seed):
    """test_titans_mlp_cuda.rs:121-560 (m_norm_max = 1.0 makes the projection bite)."""
    c = _recipe(seq_len, d, dh, s_seed=s_seed)
    y, ms, ss = gpu_forward([c], dh, act, m_norm_max)
    oy, om, os_ = orc.titans_mlp_forward(*c, dh, act, m_norm_max)
    assert_abs("y", y[0], oy, 1e-4)
    assert_abs("m_states", ms[0], om, 1e-4)
    assert_abs("s_states", ss[0], os_, 1e-4)
    if m_norm_max == 1.0:
        assert np.linalg.norm(om[1:], axis=1).max() <= 1.0 + 1e-5 and np.linalg.norm(orc.titans_mlp_forward(*c, dh, act)[1][1:], axis=1).max() > 1.0


@pytest.mark.parametrize("act,B,seq_len,d,dh", [(0, 1, 4, 8, 32), (1, 3, 6, 8, 32), (2, 2, 16, 8, 24), (0, 2, 5, 64, 128),
                                                (1, 1, 1, 8, 32)])
def test_forward_and_backward_match_oracle(act, B, seq_len, d, dh):
    chains = []
    r = np.random.default_rng(100 + act + seq_len)
    for b in range(B):
        k, v, q, alpha, theta, eta, m0, s0 = _recipe(seq_len, d, dh, seed0=42 + 10 * b, s_seed=77 + b)
        chains.append((k * 3, v * 3, q * 3, alpha, theta, eta, m0 * (2.0 / d ** 0.5 / 0.1 * 0.1), s0 * 0.1))
    dy = r.standard_normal((B, seq_len, d)).astype(f32)
    y, ms, ss = gpu_forward(chains, dh, act, F32_MAX)
    n = orc.mlp_state_size(d, dh)
    st = lambda i: dev(np.stack([c[i] for c in chains]))
    g = dict(d_k=zeros(B, seq_len, d), d_v=zeros(B, seq_len, d), d_q=zeros(B, seq_len, d), d_alpha=zeros(B, seq_len),
             d_theta=zeros(B, seq_len), d_eta=zeros(B, seq_len), d_m=dev(np.ones(n, f32)), d_s=dev(np.ones(n, f32)))
    D.call("titans_mlp_backward_f32_cuda", st(0), st(1), st(2), st(3), st(4), st(5), dev(ms), dev(ss), dev(dy),
           g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], g["d_m"], g["d_s"],
           seq_len, d, dh, B, seq_len * d, (seq_len + 1) * n, act, F32_MAX)
    torch.cuda.synchronize()
    dm_sum, ds_sum = np.zeros(n), np.zeros(n)
    for b, c in enumerate(chains):
        oy, om, os_ = orc.titans_mlp_forward(*c, dh, act)
        assert_close(f"y[{b}]", y[b], oy)
        assert_close(f"m_states[{b}]", ms[b], om)
        want = orc.titans_mlp_backward(*c[:6], om, os_, dy[b], dh, act)
        for nm in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
            assert_close(f"{nm}[{b}]", host(g[nm])[b], want[nm])
        dm_sum += want["d_m"]
        ds_sum += want["d_s"]
    assert_close("d_m_initial (summed over the batch, accumulated)", host(g["d_m"]) - 1.0, dm_sum, 2e-4)
    assert_close("d_s_initial (summed over the batch, accumulated)", host(g["d_s"]) - 1.0, ds_sum, 2e-4)
