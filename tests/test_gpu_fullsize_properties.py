"""Properties of the bf16 chunkwise path at the full size of BASELINE configs[2] (128 chains of
4096 tokens, chunk 64), beside the value check against the oracle at the same size
(test_gpu_fullsize_values.py).  The kernels contain no atomics and no data-dependent scheduling, so
each property holds bit for bit:

* chain independence: a chain's results do not depend on which other chains share the launch;
* causality: outputs and chunk states before a chunk do not depend on its tokens;
* exact scaling: the backward is linear in dY, and a factor of 2 is exact in every format on the
  path (fp32, bf16 and hi + lo pairs of bf16).

A wrong index, a race between workgroups of one chain or a dependence on launch geometry breaks
one of them."""
import pytest
import torch

from nl_hecate_amd import dispatch as D

pytestmark = pytest.mark.gpu

B, S, DH, C = 128, 4096, 64, 64
NC = S // C


def _inputs():
    g = torch.Generator(device="cuda").manual_seed(0x5EED0003)
    rn = lambda *sh: torch.randn(*sh, device="cuda", generator=g)
    k, q, v = rn(B, S, DH), rn(B, S, DH), rn(B, S, DH)
    k = k / k.norm(dim=-1, keepdim=True)
    q = q / q.norm(dim=-1, keepdim=True)
    x = dict(k=k.to(torch.bfloat16), v=v.to(torch.bfloat16), q=q.to(torch.bfloat16),
             al=torch.sigmoid(rn(B, S)), th=torch.sigmoid(rn(B, S)), et=torch.sigmoid(rn(B, S)),
             m0=0.1 * rn(B, DH, DH), s0=0.1 * rn(B, DH, DH), dy=rn(B, S, DH))
    return x


def _forward(x, sl=slice(None)):
    n = x["k"][sl].shape[0]
    z = lambda *sh: torch.zeros(*sh, device="cuda")
    mc, sc, y = z(n, NC + 1, DH, DH), z(n, NC + 1, DH, DH), z(n, S, DH)
    D.call("titans_chunkwise_forward_bf16_rocm", x["k"][sl].contiguous(), x["v"][sl].contiguous(),
           x["q"][sl].contiguous(), x["al"][sl].contiguous(), x["th"][sl].contiguous(), x["et"][sl].contiguous(),
           x["m0"][sl].contiguous(), x["s0"][sl].contiguous(), mc, sc, y, S, DH, n, C)
    return mc, sc, y


def _backward(x, mc, sc, dy, sl=slice(None)):
    n = x["k"][sl].shape[0]
    z = lambda *sh: torch.zeros(*sh, device="cuda")
    g = [z(n, S, DH), z(n, S, DH), z(n, S, DH), z(n, S), z(n, S), z(n, S), z(DH, DH), z(DH, DH)]
    D.call("titans_chunkwise_backward_bf16_rocm", x["k"][sl].contiguous(), x["v"][sl].contiguous(),
           x["q"][sl].contiguous(), x["al"][sl].contiguous(), x["th"][sl].contiguous(), x["et"][sl].contiguous(),
           mc, sc, dy, *g, S, DH, n, C)
    torch.cuda.synchronize()
    return g


def test_chains_are_independent_of_the_launch_they_share():
    x = _inputs()
    mc, sc, y = _forward(x)
    g = _backward(x, mc, sc, x["dy"])
    for sl in (slice(0, 48), slice(48, 128)):   # uneven parts: other grid sizes, other workgroup pairing
        print(f"full-size chunkwise: chains {sl.start}..{sl.stop}", flush=True)
        mc2, sc2, y2 = _forward(x, sl)
        assert torch.equal(y2, y[sl]) and torch.equal(mc2, mc[sl]) and torch.equal(sc2, sc[sl])
        g2 = _backward(x, mc2, sc2, x["dy"][sl].contiguous(), sl)
        for a, b in zip(g2[:6], g[:6]):   # per-chain gradients; d_m_initial / d_s_initial sum over chains
            assert torch.equal(a, b[sl])
    assert all(torch.isfinite(t).all() for t in g)


def test_forward_is_causal_across_chunks():
    x = _inputs()
    mc, sc, y = _forward(x)
    cut = 40 * C   # tokens from chunk 40 on are replaced
    x2 = dict(x)
    for n in ("k", "v", "q"):
        x2[n] = x[n].clone()
        x2[n][:, cut:] = x[n][:, cut:].flip(1)
    for n in ("al", "th", "et"):
        x2[n] = x[n].clone()
        x2[n][:, cut:] = 1.0 - x[n][:, cut:]
    mc2, sc2, y2 = _forward(x2)
    assert torch.equal(y2[:, :cut], y[:, :cut])
    assert torch.equal(mc2[:, :41], mc[:, :41]) and torch.equal(sc2[:, :41], sc[:, :41])
    assert not torch.equal(y2[:, cut:], y[:, cut:])


def test_backward_scales_exactly_with_the_upstream_gradient():
    x = _inputs()
    mc, sc, _ = _forward(x)
    g1 = _backward(x, mc, sc, x["dy"])
    g2 = _backward(x, mc, sc, 2.0 * x["dy"])
    for a, b in zip(g1, g2):
        assert torch.equal(2.0 * a, b)
