"""GPU parity of the frozen-M0 chunkwise rules (Titans / Delta) through the
reference's entry-point names against the CPU oracle.  fp32 path: relative
tolerance 1e-4 (max|a-b|/max|b|)."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu
F32_MAX = orc.F32_MAX


def oracle_chunkwise(x, C, has_s, clip=0.0, mx=F32_MAX):
    B = x["k"].shape[0]
    fw, bw = [], []
    for b in range(B):
        a = [x[n][b] for n in ("k", "v", "q", "alpha", "theta", "eta")]
        y, mc, sc = orc.chunkwise_forward(*a, x["m0"][b], x["s0"][b], C, has_s, clip, mx)
        fw.append((y, mc, sc))
        bw.append(orc.chunkwise_backward(*a, mc, sc, x["dy"][b], C, has_s, clip, mx))
    out = dict(y=np.stack([f[0] for f in fw]), mc=np.stack([f[1] for f in fw]),
               sc=np.stack([f[2] for f in fw]))
    g = {n: np.stack([o[n] for o in bw]) for n in bw[0] if n not in ("d_m", "d_s")}
    g["d_m_initial"] = sum(o["d_m"] for o in bw)
    g["d_s_initial"] = sum(o["d_s"] for o in bw)
    if not has_s:
        g.pop("d_eta"); g.pop("d_s_initial")
    return out, g


def gpu_chunkwise(x, C, has_s, clip=0.0, mx=F32_MAX):
    B, s, d = x["k"].shape
    nc = (s + C - 1) // C
    k, v, q, dy = dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["dy"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    mc, sc, y = zeros(B, nc + 1, d, d), zeros(B, nc + 1, d, d), zeros(B, s, d)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_m_initial=zeros(d, d))
    if has_s:
        g.update(d_eta=zeros(B, s), d_s_initial=zeros(d, d))
        D.call("titans_chunkwise_forward_f32_cuda", k, v, q, al, th, et, dev(x["m0"]), dev(x["s0"]),
               mc, sc, y, s, d, B, C, clip, mx)
        D.call("titans_chunkwise_backward_f32_cuda", k, v, q, al, th, et, mc, sc, dy,
               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
               g["d_m_initial"], g["d_s_initial"], s, d, B, C, clip, mx)
    else:
        D.call("delta_chunkwise_forward_f32_cuda", k, v, q, al, th, dev(x["m0"]), mc, y,
               s, d, B, C, clip, mx)
        D.call("delta_chunkwise_backward_f32_cuda", k, v, q, al, th, mc, dy,
               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_m_initial"],
               s, d, B, C, clip, mx)
    torch.cuda.synchronize()
    return dict(y=host(y), mc=host(mc), sc=host(sc)), {n: host(t) for n, t in g.items()}


@pytest.mark.parametrize("has_s", [True, False])
@pytest.mark.parametrize("B,s,d,C", [(3, 192, 64, 64), (2, 100, 64, 64), (2, 70, 64, 16), (3, 40, 16, 8),
                                     (2, 50, 32, 32), (2, 40, 128, 16), (2, 150, 64, 100), (2, 30, 8, 4),
                                     (2, 23, 64, 5)])
def test_chunkwise_forward_backward_parity(has_s, B, s, d, C):
    x = rule_inputs(B, s, d, 9000 + s + d + C, m0_scale=0.2)
    f, g = gpu_chunkwise(x, C, has_s)
    fo, go = oracle_chunkwise(x, C, has_s)
    assert_close("y", f["y"], fo["y"])
    assert_close("m_chunk_states", f["mc"], fo["mc"])
    if has_s:
        assert_close("s_chunk_states", f["sc"], fo["sc"])
    for n in go:
        assert_close(n, g[n], go[n])


@pytest.mark.parametrize("clip,mx", [(0.7, F32_MAX), (0.0, 1.5), (0.7, 1.5)])
def test_chunkwise_with_clip_and_projection(clip, mx):
    x = rule_inputs(2, 48, 64, 9100, m0_scale=0.3)
    x["v"] *= 2.0
    f, g = gpu_chunkwise(x, 16, True, clip, mx)
    fo, go = oracle_chunkwise(x, 16, True, clip, mx)
    assert_close("y", f["y"], fo["y"])
    for n in go:
        assert_close(n, g[n], go[n])


def test_chunk_size_one_is_the_exact_rule():
    """core/src/gpu_forward.rs:4193-4338: C=1 reproduces the per-token kernels."""
    B, s, d = 3, 37, 64
    x = rule_inputs(B, s, d, 9200, m0_scale=0.2)
    f, g = gpu_chunkwise(x, 1, True)
    ms, ss, y = zeros(B, s + 1, d, d), zeros(B, s + 1, d, d), zeros(B, s, d)
    D.titans_forward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                        dev(x["eta"]), dev(x["m0"]), dev(x["s0"]), ms, ss, y, s, d, B, s, d * d,
                        0.0, F32_MAX)
    torch.cuda.synchronize()
    assert_close("y", f["y"], host(y), 1e-5)
    assert_close("M", f["mc"], host(ms), 1e-5)
    assert_close("S", f["sc"], host(ss), 1e-5)


def test_chunkwise_differs_from_exact_for_larger_chunks():
    x = rule_inputs(2, 64, 64, 9300, m0_scale=0.2)
    f, _ = gpu_chunkwise(x, 16, True)
    yo, _, _ = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                        x["m0"], x["s0"])
    assert np.abs(f["y"] - yo).max() > 1e-3
