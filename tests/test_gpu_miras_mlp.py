"""GPU parity of the MIRAS MLP memories MONETA and YAAD through the C ABI against the CPU oracle (relative 1e-4):
every error function (l_2, l_1, general l_p, Huber on both sides of delta), L_q normalisation in the forward,
boundary snapshots, hidden sizes that are not powers of two, and the accumulate contract of d_k / d_v."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
f32 = np.float32


def _inputs(s, d, dh, seed):
    r = np.random.default_rng(seed)
    k, v, q, dy = (r.standard_normal((s, d)).astype(f32) for _ in range(4))
    sig = lambda x: 1 / (1 + np.exp(-x))
    alpha = (0.8 + 0.19 * sig(r.standard_normal(s))).astype(f32)
    theta = (0.1 * sig(r.standard_normal(s))).astype(f32)
    w1 = (r.standard_normal((dh, d)) / d ** 0.5).astype(f32)
    w2 = (r.standard_normal((d, dh)) / dh ** 0.5).astype(f32)
    bnd = ((w1 + 0.1 * r.standard_normal((dh, d))).astype(f32), (w2 + 0.1 * r.standard_normal((d, dh))).astype(f32))
    return k, v, q, alpha, theta, w1, w2, bnd, dy


@pytest.mark.parametrize("mode,p1,p2,lq,s,d,dh", [(0, 2.0, 10.0, 2.0, 12, 8, 16), (0, 1.0, 3.0, 2.0, 9, 8, 24),
                                                 (0, 1.5, 3.0, 2.0, 7, 16, 40), (0, 2.0, 10.0, 3.0, 6, 8, 16),
                                                 (1, 0.5, 0.05, 2.0, 12, 8, 16), (1, 0.5, 0.0, 2.0, 5, 64, 128),
                                                 (0, 2.0, 10.0, 2.0, 1, 8, 16)])
def test_forward_and_backward_match_oracle(mode, p1, p2, lq, s, d, dh):
    k, v, q, alpha, theta, w1, w2, bnd, dy = _inputs(s, d, dh, 7 + s + dh)
    lam2 = 0.01
    w1s, w2s, y = zeros(s + 1, dh, d), zeros(s + 1, d, dh), zeros(s, d)
    if mode == 0:
        D.call("mlp_forward_lp_f32_cuda", dev(k), dev(v), dev(q), dev(alpha), dev(theta), dev(w1), dev(w2), w1s, w2s, y,
               s, d, dh, p1, p2, lam2, lq)
        boundary = None
    else:
        D.call("mlp_forward_huber_f32_cuda", dev(k), dev(v), dev(q), dev(alpha), dev(theta), dev(w1), dev(w2),
               dev(bnd[0]), dev(bnd[1]), w1s, w2s, y, s, d, dh, p1, p2, lam2)
        boundary = bnd
    torch.cuda.synchronize()
    oy, o1, o2 = orc.miras_mlp_forward(mode, k, v, q, alpha, theta, w1, w2, dh, p1, p2, lam2, lq, boundary)
    assert_close("y", host(y), oy)
    assert_close("w1_states", host(w1s), o1)
    assert_close("w2_states", host(w2s), o2)
    if lq != 2.0:
        return   # the backward covers q = 2 only (moneta_backward.cu:547-552)
    g = dict(d_k=dev(np.full((s, d), 0.5, f32)), d_v=dev(np.full((s, d), -0.25, f32)), d_q=zeros(s, d),
             d_alpha=zeros(s), d_theta=zeros(s), d_w1=dev(np.full((dh, d), 9.0, f32)), d_w2=dev(np.full((d, dh), 9.0, f32)))
    if mode == 0:
        D.call("mlp_backward_lp_f32_cuda", dev(k), dev(v), dev(q), dev(alpha), dev(theta), dev(o1), dev(o2), dev(dy),
               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_w1"], g["d_w2"], s, d, dh, p1, p2, lam2, 2.0)
    else:
        D.call("mlp_backward_huber_f32_cuda", dev(k), dev(v), dev(q), dev(alpha), dev(theta), dev(o1), dev(o2),
               dev(bnd[0]), dev(bnd[1]), dev(dy), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_w1"],
               g["d_w2"], s, d, dh, p1, p2, lam2)
    torch.cuda.synchronize()
    want = orc.miras_mlp_backward(mode, k, v, q, alpha, theta, o1, o2, dy, dh, p1, p2, lam2, boundary)
    assert_close("d_k (added to)", host(g["d_k"]) - 0.5, want["d_k"])
    assert_close("d_v (subtracted from)", host(g["d_v"]) + 0.25, want["d_v"])
    for nm in ("d_q", "d_alpha", "d_theta", "d_w1", "d_w2"):   # written, not accumulated
        assert_close(nm, host(g[nm]), want[nm])
