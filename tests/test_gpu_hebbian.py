"""GPU parity of the Hebbian rule (M <- (1 - alpha) M + v k^T) through the C ABI against the CPU oracle:
the reference's own test recipes (core/tests/test_cuda_hebbian.rs: rand_buf seeds, alpha = 0.05, absolute
1e-5 forward / 1e-4 backward), config-shaped batches at every supported head size with the kernels' stride
contract, and the checkpoint / segment composition.  Tolerance elsewhere: relative 1e-4 (fp32 path)."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_abs, assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu


def gpu_forward(k, v, q, alpha, m0, input_stride=None, m_stride=None, s=None):
    B, d = k.shape[0], k.shape[2]
    s = k.shape[1] if s is None else s
    ms, y = zeros(B, s + 1, d, d), zeros(B, s, d)
    D.hebbian_forward_dd(dev(k), dev(v), dev(q), dev(alpha), dev(m0), ms, y, s, d, B,
                         input_stride or s, m_stride or d * d)
    torch.cuda.synchronize()
    return host(y), host(ms)


def oracle_forward(k, v, q, alpha, m0):
    out = [orc.hebbian_forward(k[b], v[b], q[b], alpha[b], m0[b]) for b in range(k.shape[0])]
    return np.stack([o[0] for o in out]), np.stack([o[1] for o in out])


def _recipe(seq_len, d, seeds):
    rb = lambda n, seed: orc.simple_rng_uniform(n, seed)
    k, v, q = (rb(seq_len * d, sd).reshape(1, seq_len, d) for sd in seeds[:3])
    alpha = np.full((1, seq_len), 0.05, np.float32)
    return k, v, q, alpha


@pytest.mark.parametrize("seq_len,d,seeds,m0_seed", [(16, 8, (100, 200, 300), None), (1, 8, (400, 500, 600), None),
                                                    (8, 8, (700, 800, 900), 1000), (8, 16, (3000, 3100, 3200), None),
                                                    (4, 128, (5000, 5100, 5200), None)])
def test_reference_forward_recipes(seq_len, d, seeds, m0_seed):
    """test_cuda_hebbian.rs:53-126, 274-330."""
    k, v, q, alpha = _recipe(seq_len, d, seeds)
    m0 = np.zeros((1, d, d), np.float32) if m0_seed is None else orc.simple_rng_uniform(d * d, m0_seed).reshape(1, d, d)
    y, ms = gpu_forward(k, v, q, alpha, m0)
    yo, mo = oracle_forward(k, v, q, alpha, m0)
    assert_abs("y", y, yo, 1e-5)
    assert_abs("m_states", ms, mo, 1e-5)
    assert np.linalg.norm(ms[0, -1]) > 1e-6


def test_reference_backward_recipe():
    """test_cuda_hebbian.rs:128-207: d = 8, 12 tokens, zero M_0."""
    s, d = 12, 8
    k, v, q, alpha = _recipe(s, d, (1100, 1200, 1300))
    dy = orc.simple_rng_uniform(s * d, 1400).reshape(s, d)
    _, mo = orc.hebbian_forward(k[0], v[0], q[0], alpha[0], np.zeros((d, d), np.float32))
    want = orc.hebbian_backward(k[0], v[0], q[0], alpha[0], mo, dy)
    g = dict(d_k=zeros(s, d), d_v=zeros(s, d), d_q=zeros(s, d), d_alpha=zeros(s), d_m=torch.full((d, d), 7.0, device="cuda"))
    D.hebbian_backward_dd(dev(k[0]), dev(v[0]), dev(q[0]), dev(alpha[0]), dev(mo), dev(dy),
                          g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_m"], s, d)
    torch.cuda.synchronize()
    for n in want:   # d_m_initial is overwritten (hebbian_backward.cu:277-280)
        assert_abs(n, host(g[n]), want[n], 1e-4)


@pytest.mark.parametrize("B,s,d", [(3, 40, 16), (5, 33, 32), (6, 70, 64), (3, 257, 64), (2, 64, 64), (2, 129, 64), (1, 1000, 64), (2, 9, 128),
                                   (2, 21, 8)])
def test_batched_forward_and_segment_backward_match_oracle(B, s, d):
    x = rule_inputs(B, s, d, 900 + d + s, m0_scale=0.3)
    y, ms = gpu_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
    yo, mo = oracle_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    # whole sequence as one segment, seeded: every chain against the single-chain oracle
    seed = 0.1 * np.random.default_rng(5).standard_normal((B, d, d)).astype(np.float32)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s), d_m=zeros(B, d, d))
    D.hebbian_backward_dd_segment(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(mo), dev(x["dy"]),
                                  dev(seed), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_m"], 0, s, d, B, s)
    torch.cuda.synchronize()
    for b in range(B):
        want = orc.hebbian_backward(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], mo[b], x["dy"][b], d_m_seed=seed[b])
        for n in want:
            assert_close(f"{n}[{b}]", host(g[n])[b], want[n])


@pytest.mark.parametrize("B,S,s,d", [(3, 24, 10, 16), (2, 300, 200, 64)])
def test_forward_strides_select_a_window_of_a_longer_sequence(B, S, s, d):
    """input_stride / m_stride as in the other rules' forwards (core/kernels/hebbian_forward.cu:75-90)."""
    x = rule_inputs(B, S, d, 77, m0_scale=0.2)
    pool = np.concatenate([x["m0"], x["s0"]], 1).reshape(B, 2 * d * d)   # states with stride 2 d^2
    y, ms = gpu_forward(x["k"], x["v"], x["q"], x["alpha"], pool, input_stride=S, m_stride=2 * d * d, s=s)
    yo, mo = oracle_forward(x["k"][:, :s], x["v"][:, :s], x["q"][:, :s], x["alpha"][:, :s], x["m0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)


@pytest.mark.parametrize("s,d,C", [(23, 32, 4), (23, 32, 7), (23, 32, 64), (150, 64, 64), (150, 64, 100),
                                   (150, 64, 9)])
def test_checkpointed_forward_and_segment_backward_compose(s, d, C):
    x = rule_inputs(1, s, d, 31, m0_scale=0.3)
    k, v, q, alpha, m0, dy = (x[n][0] for n in ("k", "v", "q", "alpha", "m0", "dy"))
    yo, ck = orc.hebbian_forward(k, v, q, alpha, m0, checkpoint_interval=C)
    n = ck.shape[0]
    ckg, y = zeros(n, d, d), zeros(s, d)
    D.hebbian_forward_dd_ckpt(dev(k), dev(v), dev(q), dev(alpha), dev(m0), ckg, y, s, d, C)
    torch.cuda.synchronize()
    assert_close("y", host(y), yo)
    assert_close("checkpoints", host(ckg), ck)
    _, mo = orc.hebbian_forward(k, v, q, alpha, m0)
    want = orc.hebbian_backward(k, v, q, alpha, mo, dy)
    ends = [t + 1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s]
    starts = [0] + ends[:-1]
    g = dict(d_k=zeros(1, s, d), d_v=zeros(1, s, d), d_q=zeros(1, s, d), d_alpha=zeros(1, s))
    seed = zeros(1, d, d)
    kd, vd, qd, ad, dyd = (dev(t[None]) for t in (k, v, q, alpha, dy))
    for i in reversed(range(len(ends))):
        lo, hi = starts[i], ends[i]
        local, yl = zeros(1, hi - lo + 1, d, d), zeros(1, hi - lo, d)
        D.hebbian_forward_dd(kd[:, lo:], vd[:, lo:], qd[:, lo:], ad[:, lo:], ckg[i:i + 1], local, yl,
                             hi - lo, d, 1, s, d * d)   # replay from the checkpoint
        out = zeros(1, d, d)
        D.hebbian_backward_dd_segment(kd, vd, qd, ad, local, dyd, seed, g["d_k"], g["d_v"], g["d_q"], g["d_alpha"],
                                      out, lo, hi, d, 1, s)
        seed = out
    torch.cuda.synchronize()
    for n in g:
        assert_close(n, host(g[n])[0], want[n])
    assert_close("d_m", host(seed)[0], want["d_m"])


@pytest.mark.parametrize("d", [32, 64])
def test_saturated_gates(d):
    """alpha = 1 wipes the memory (retention 0) and alpha = 0 keeps it: the gradient of a wiped step still
    depends on the state before it, so nothing in the backward may divide by the retention."""
    B, s = 2, 150
    x = rule_inputs(B, s, d, 4242, m0_scale=0.3)
    x["alpha"][:, 5::17] = 1.0
    x["alpha"][:, 9::23] = 0.0
    x["alpha"][0, 63] = 1.0   # last token of a 64-token chunk
    x["alpha"][1, 64] = 1.0   # first token of the next one
    y, ms = gpu_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
    yo, mo = oracle_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s), d_m=zeros(B, d, d))
    D.hebbian_backward_dd_segment(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(mo), dev(x["dy"]),
                                  None, g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_m"], 0, s, d, B, s)
    torch.cuda.synchronize()
    for b in range(B):
        want = orc.hebbian_backward(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], mo[b], x["dy"][b])
        for n in want:
            assert_close(f"{n}[{b}]", host(g[n])[b], want[n])
