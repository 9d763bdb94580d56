"""GPU parity of the phase-2 kernels (per-chunk recurrence / reverse sweep with the errors
supplied by the caller) against the numpy oracle, and — driven chunk by chunk with errors
computed from the chunk-start state — against the chunkwise oracle they are a piece of.
fp32: relative 1e-4."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu
F32_MAX = orc.F32_MAX


def run_chunks(x, C, titans, m_norm_max=F32_MAX, clip=0.0):
    """Forward then backward over all chunks through the phase-2 entry points; the errors of a
    chunk are pred - v with pred = K M0^T (torch matmul stands in for the caller's GEMM)."""
    B, s, d = x["k"].shape
    nc = (s + C - 1) // C
    k, v, q, dy = dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["dy"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    m_work, s_work = dev(x["m0"]).clone(), dev(x["s0"]).clone()
    mc, sc, y = zeros(B, nc + 1, d, d), zeros(B, nc + 1, d, d), zeros(B, s, d)
    errs = []
    for ci in range(nc):
        t0, t1 = ci * C, min(s, ci * C + C)
        pred = zeros(B, C, d)
        pred[:, :t1 - t0] = torch.einsum("btj,bij->bti", k[:, t0:t1], m_work)
        vv = zeros(B, C, d)
        vv[:, :t1 - t0] = v[:, t0:t1]
        D.call("error_subtract_clip_f32_cuda", pred, vv, B * C, d, clip)
        errs.append(pred)
        if titans:
            D.call("titans_phase2_forward_f32_cuda", k, q, al, th, et, pred, m_work, s_work, mc, sc, y,
                   s, d, B, C, ci, m_norm_max)
        else:
            D.call("delta_phase2_forward_f32_cuda", k, q, al, th, pred, m_work, mc, y, s, d, B, C, ci, m_norm_max)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_eta=zeros(B, s))
    dM, dS, dM0 = zeros(B, d, d), zeros(B, d, d), zeros(B, d, d)
    mrec, srec = zeros(B, C + 1, d, d), zeros(B, C + 1, d, d)
    for ci in range(nc - 1, -1, -1):
        if titans:
            D.call("titans_phase2_backward_f32_cuda", k, q, al, th, et, errs[ci], mc, sc, dy, g["d_k"], g["d_v"],
                   g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], dM, dS, dM0, mrec, srec, s, d, B, C, ci,
                   m_norm_max)
        else:
            D.call("delta_phase2_backward_f32_cuda", k, q, al, th, errs[ci], mc, dy, g["d_k"], g["d_v"], g["d_q"],
                   g["d_alpha"], g["d_theta"], dM, dM0, mrec, s, d, B, C, ci, m_norm_max)
    torch.cuda.synchronize()
    out = {n: host(t) for n, t in g.items()}
    out.update(y=host(y), mc=host(mc), sc=host(sc), d_m=host(dM), d_s=host(dS))
    return out


@pytest.mark.parametrize("titans", [True, False])
@pytest.mark.parametrize("B,s,d,C", [(2, 48, 64, 16), (3, 37, 32, 8), (2, 20, 16, 20), (2, 64, 64, 64)])
def test_phase2_chain_equals_chunkwise_oracle(titans, B, s, d, C):
    x = rule_inputs(B, s, d, seed=s + d + C, m0_scale=0.1)
    if not titans:
        x["s0"][:] = 0
    got = run_chunks(x, C, titans)
    for b in range(B):
        a = [x[n][b] for n in ("k", "v", "q", "alpha", "theta", "eta")]
        y, mc, sc = orc.chunkwise_forward(*a, x["m0"][b], x["s0"][b], C, titans)
        w = orc.chunkwise_backward(*a, mc, sc, x["dy"][b], C, titans)
        assert_close("y", got["y"][b], y)
        assert_close("m_chunk_states", got["mc"][b], mc)
        if titans:
            assert_close("s_chunk_states", got["sc"][b], sc)
        for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta") + (("d_eta",) if titans else ()):
            assert_close(n, got[n][b], w[n])
        assert_close("d_M", got["d_m"][b], w["d_m"])
        if titans:
            assert_close("d_S", got["d_s"][b], w["d_s"])


@pytest.mark.parametrize("titans", [True, False])
def test_phase2_with_arbitrary_errors_and_projection(titans):
    """Errors that are NOT M0 k - v (the kernels must take them as given), M-norm projection on,
    nonzero incoming adjoints: against the numpy restatement."""
    B, s, d, C, ci = 2, 40, 32, 16, 1
    r = np.random.default_rng(5)
    f = np.float32
    x = rule_inputs(B, s, d, seed=11, m0_scale=0.3)
    errors = r.standard_normal((B, C, d)).astype(f)
    m_in, s_in = x["m0"], (x["s0"] if titans else np.zeros_like(x["s0"]))
    dM_in, dS_in = (0.2 * r.standard_normal((B, d, d)).astype(f) for _ in range(2))
    mx = 2.0
    nc = (s + C - 1) // C
    k, q, dy = dev(x["k"]), dev(x["q"]), dev(x["dy"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    m_work, s_work = dev(m_in).clone(), dev(s_in).clone()
    mc, sc, y = zeros(B, nc + 1, d, d), zeros(B, nc + 1, d, d), zeros(B, s, d)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_eta=zeros(B, s))
    dM, dS, dM0 = dev(dM_in).clone(), dev(dS_in).clone(), zeros(B, d, d)
    mrec, srec = zeros(B, C + 1, d, d), zeros(B, C + 1, d, d)
    if titans:
        D.call("titans_phase2_forward_f32_cuda", k, q, al, th, et, dev(errors), m_work, s_work, mc, sc, y, s, d, B,
               C, ci, mx)
        D.call("titans_phase2_backward_f32_cuda", k, q, al, th, et, dev(errors), mc, sc, dy, g["d_k"], g["d_v"],
               g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], dM, dS, dM0, mrec, srec, s, d, B, C, ci, mx)
    else:
        D.call("delta_phase2_forward_f32_cuda", k, q, al, th, dev(errors), m_work, mc, y, s, d, B, C, ci, mx)
        D.call("delta_phase2_backward_f32_cuda", k, q, al, th, dev(errors), mc, dy, g["d_k"], g["d_v"], g["d_q"],
               g["d_alpha"], g["d_theta"], dM, dM0, mrec, s, d, B, C, ci, mx)
    torch.cuda.synchronize()
    sl = slice(ci * C, ci * C + C)
    for b in range(B):
        eta = x["eta"][b, sl] if titans else None
        yw, mw, sw = orc.phase2_forward(x["k"][b, sl], x["q"][b, sl], x["alpha"][b, sl], x["theta"][b, sl], eta,
                                        errors[b], m_in[b], s_in[b], mx)
        assert_close("y", host(y)[b, sl], yw)
        assert_close("m_work", host(m_work)[b], mw)
        assert np.linalg.norm(host(m_work)[b]) <= mx * (1 + 1e-5)
        assert_close("chunk-start slot", host(mc)[b, ci], m_in[b], 1e-7)
        w = orc.phase2_backward(x["k"][b, sl], x["q"][b, sl], x["alpha"][b, sl], x["theta"][b, sl], eta, errors[b],
                                m_in[b], s_in[b], x["dy"][b, sl], dM_in[b], dS_in[b], mx)
        for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta") + (("d_eta",) if titans else ()):
            assert_close(n, host(g[n])[b, sl], w[n])
        assert_close("d_M", host(dM)[b], w["d_m"])
        assert_close("d_M0", host(dM0)[b], w["d_m0"])
        if titans:
            assert_close("d_S", host(dS)[b], w["d_s"])
