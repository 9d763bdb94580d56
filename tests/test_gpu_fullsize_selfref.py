"""Properties of the HOPE self-referential path at the launch size of BASELINE configs[3] (values
against the oracle at that size: test_gpu_fullsize_values.py).  configs[3] is 64 chains of 2048 tokens = 2048 chunks of
64 tokens; with its distributions (x ~ N(0, 1/d), so alpha = sigmoid(~0) = 1/2 at every token) every
memory halves per token and is exactly zero in fp32 after about 150 tokens, in the reference's
equations as here, so all later chunks of a chain carry zeros.  To keep every chunk's data alive the
same 2048 chunks are arranged as 1024 chains of 128 tokens.  The kernels contain no atomics and no
data-dependent scheduling, so each property holds bit for bit:

* chain independence: a chain's outputs, caches and gradients do not depend on which other
  chains share the launch (other grid sizes for all four kernels);
* causality: outputs, caches and snapshots before a chunk do not depend on its tokens;
* exact scaling: the backward is linear in dY and a factor of 2 is exact in fp32 (above the
  underflow threshold).

Small sizes against the oracle: test_gpu_selfref.py."""
import pytest
import torch

from nl_hecate_amd import selfref as SR

pytestmark = pytest.mark.gpu

B, S, DH, C = 1024, 128, 64, 64


def _inputs():
    g = torch.Generator(device="cuda").manual_seed(0x5EED0004)
    lim = (6.0 / (2 * DH)) ** 0.5
    # all six memories Xavier-uniform: with self-generated values a zero M_mem stays zero (its error is
    # F_mem (k - v)), which would leave y, d_x and five of the six memory gradients identically zero
    mems = (torch.rand(B, 6, DH, DH, device="cuda", generator=g) * 2 - 1) * lim
    x = torch.randn(B, S, DH, device="cuda", generator=g) / (8 * DH) ** 0.5
    dy = torch.randn(B, S, DH, device="cuda", generator=g)
    return mems, x, dy


CACHE_FIELDS = ("k_mem", "v_mem", "q_mem", "alpha", "theta", "alpha_mean", "eta_mean", "frozen_snapshots")


def _run(mems, x, dy, sl=slice(None), scale=1.0):
    m = mems[sl].clone()
    y, c = SR.chunkwise_self_ref_step(m, x[sl].contiguous(), C, True)
    d_emb, d_mems = SR.chunkwise_self_ref_step_backward(c, (scale * dy[sl]).contiguous())
    torch.cuda.synchronize()
    return dict(y=y, mems=m, d_emb=d_emb, d_mems=d_mems, **{n: getattr(c, n) for n in CACHE_FIELDS})


def test_chains_are_independent_of_the_launch_they_share():
    mems, x, dy = _inputs()
    full = _run(mems, x, dy)
    assert all(torch.isfinite(t).all() for t in full.values())
    assert float(full["y"][:, C:C + 16].abs().max()) > 0 and float(full["d_emb"][:, :C].abs().max()) > 0
    for sl in (slice(0, 300), slice(300, 1024)):
        print(f"full-size self-referential step: chains {sl.start}..{sl.stop}", flush=True)
        part = _run(mems, x, dy, sl)
        for n, t in part.items():
            assert torch.equal(t, full[n][sl]), n


def test_forward_is_causal_across_chunks():
    mems, x, dy = _inputs()
    a = _run(mems, x, dy)
    cut = C
    x2 = x.clone()
    x2[:, cut:] = x[:, cut:].flip(1)
    b = _run(mems, x2, dy)
    for n in ("y", "k_mem", "v_mem", "q_mem", "alpha", "theta", "alpha_mean", "eta_mean"):
        assert torch.equal(a[n][:, :cut], b[n][:, :cut]), n
    assert torch.equal(a["frozen_snapshots"][:, :2], b["frozen_snapshots"][:, :2])
    assert not torch.equal(a["k_mem"][:, cut:], b["k_mem"][:, cut:])


def test_backward_scales_exactly_with_the_upstream_gradient():
    """Doubling dY doubles every gradient exactly, except where a value sits at the underflow
    threshold of fp32 (the memories decay by 2^-128 over a chain): there 2 * flush(x) and flush(2 x)
    may differ, so elements below 1e-30 are compared with an absolute bound instead."""
    mems, x, dy = _inputs()
    a = _run(mems, x, dy)
    b = _run(mems, x, dy, scale=2.0)
    for n in ("d_emb", "d_mems"):
        big = a[n].abs() >= 1e-30
        assert torch.equal((2.0 * a[n])[big], b[n][big]), n
        assert float(((2.0 * a[n] - b[n]).abs() * (~big)).max()) < 1e-29, n
