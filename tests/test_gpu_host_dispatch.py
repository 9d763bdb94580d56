"""GPU parity of the host-slice dispatch layer (`nlh_*_dispatch`, the bodies of
the reference's `*_dispatch` functions, core/src/dispatch.rs:378-460, 746-895,
1083-1224) against the CPU oracle: one chain, numpy slices in and out, the way a
rule struct or an opaque VJP block of the tape calls them.

Tolerances: rel 1e-4 (max|a-b| / max|b|) for the float rules; 2e-2 for
sliding-window attention, whose operands and stored weights are bf16.
"""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tests.gpu_util import REL_TOL_BF16, REL_TOL_F32, rule_inputs

pytestmark = pytest.mark.gpu

F32_MAX = float(np.finfo(np.float32).max)


def relerr(a, b):
    return float(np.max(np.abs(a - b)) / max(float(np.max(np.abs(b))), 1e-30))


def z(*shape):
    return np.zeros(shape, np.float32)


SHAPES = [(12, 8), (33, 64), (70, 32)]


@pytest.mark.parametrize("s,d", SHAPES)
@pytest.mark.parametrize("rule", ["delta", "dgd"])
def test_delta_and_dgd_dispatch_match_oracle(rule, s, d):
    from nl_hecate_amd import host_dispatch as H
    x = {n: a[0] for n, a in rule_inputs(1, s, d, seed=100 + s + d, m0_scale=0.1).items()}
    clip = 0.0 if rule == "delta" else 1.5
    m_states, y = z(s + 1, d, d), z(s, d)
    if rule == "delta":
        H.delta_forward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"], m_states, y, s, d, clip, F32_MAX)
    else:
        H.dgd_forward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"], m_states, y, s, d, clip)
    y_ref, ms_ref = orc.delta_forward(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"], error_clip=clip)
    assert relerr(y, y_ref) < REL_TOL_F32
    assert relerr(m_states, ms_ref) < REL_TOL_F32
    g = dict(d_k=z(s, d), d_v=z(s, d), d_q=z(s, d), d_alpha=z(s), d_theta=z(s), d_m=z(d, d))
    fn = H.delta_backward_dispatch if rule == "delta" else H.dgd_backward_dispatch
    fn(x["k"], x["v"], x["q"], x["alpha"], x["theta"], ms_ref, x["dy"], g["d_k"], g["d_v"], g["d_q"],
       g["d_alpha"], g["d_theta"], g["d_m"], s, d, clip)
    ref = orc.delta_backward(x["k"], x["v"], x["q"], x["alpha"], x["theta"], ms_ref, x["dy"], error_clip=clip)
    for n in g:
        assert relerr(g[n], ref[n]) < REL_TOL_F32, n


@pytest.mark.parametrize("s,d", SHAPES)
def test_titans_dispatch_matches_oracle(s, d):
    from nl_hecate_amd import host_dispatch as H
    x = {n: a[0] for n, a in rule_inputs(1, s, d, seed=200 + s + d, m0_scale=0.1).items()}
    m_states, s_states, y = z(s + 1, d, d), z(s + 1, d, d), z(s, d)
    H.titans_forward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], x["m0"], x["s0"],
                              m_states, s_states, y, s, d, 0.0, F32_MAX)
    y_ref, ms_ref, ss_ref = orc.titans_forward(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                               x["m0"], x["s0"])
    assert relerr(y, y_ref) < REL_TOL_F32
    assert relerr(m_states, ms_ref) < REL_TOL_F32 and relerr(s_states, ss_ref) < REL_TOL_F32
    g = dict(d_k=z(s, d), d_v=z(s, d), d_q=z(s, d), d_alpha=z(s), d_theta=z(s), d_eta=z(s), d_m=z(d, d), d_s=z(d, d))
    H.titans_backward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], ms_ref, ss_ref, x["dy"],
                               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], g["d_m"],
                               g["d_s"], s, d, 0.0)
    ref = orc.titans_backward(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], ms_ref, ss_ref, x["dy"])
    for n in g:
        assert relerr(g[n], ref[n]) < REL_TOL_F32, n


@pytest.mark.parametrize("s,d", SHAPES)
def test_hebbian_dispatch_matches_oracle(s, d):
    from nl_hecate_amd import host_dispatch as H
    x = {n: a[0] for n, a in rule_inputs(1, s, d, seed=300 + s + d, m0_scale=0.1).items()}
    m_states, y = z(s + 1, d, d), z(s, d)
    H.hebbian_forward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["m0"], m_states, y, s, d, F32_MAX)
    y_ref, ms_ref = orc.hebbian_forward(x["k"], x["v"], x["q"], x["alpha"], x["m0"])
    assert relerr(y, y_ref) < REL_TOL_F32 and relerr(m_states, ms_ref) < REL_TOL_F32
    g = dict(d_k=z(s, d), d_v=z(s, d), d_q=z(s, d), d_alpha=z(s), d_m=z(d, d))
    H.hebbian_backward_dispatch(x["k"], x["v"], x["q"], x["alpha"], ms_ref, x["dy"], g["d_k"], g["d_v"], g["d_q"],
                                g["d_alpha"], g["d_m"], s, d)
    ref = orc.hebbian_backward(x["k"], x["v"], x["q"], x["alpha"], ms_ref, x["dy"])
    for n in g:
        assert relerr(g[n], ref[n]) < REL_TOL_F32, n


def test_hebbian_dispatch_refuses_the_clamped_case():
    """dispatch.rs:1096-1105 sends 0 < m_norm_max < f32::MAX to the CPU loops; this library has none."""
    from nl_hecate_amd import host_dispatch as H
    from nl_hecate_amd.ffi import lib
    s, d = 4, 8
    x = {n: a[0] for n, a in rule_inputs(1, s, d, seed=7).items()}
    lib.nlh_set_error_mode(1)
    try:
        H.hebbian_forward_dispatch(x["k"], x["v"], x["q"], x["alpha"], x["m0"], z(s + 1, d, d), z(s, d), s, d, 2.0)
        msg = lib.nlh_last_error()
        assert msg and b"clamp" in msg
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)


@pytest.mark.parametrize("s,H_,hd,ws", [(40, 2, 32, 16), (130, 4, 64, 64)])
def test_swa_dispatch_matches_oracle(s, H_, hd, ws):
    from nl_hecate_amd import host_dispatch as H
    r = np.random.default_rng(400 + s)
    f = np.float32
    q, k, v = (r.standard_normal((s, H_ * hd)).astype(f) * 0.5 for _ in range(3))
    d_out = r.standard_normal((s, H_ * hd)).astype(f)
    out, aw = z(s, H_ * hd), z(H_, s, ws)
    H.swa_forward_dispatch(q, k, v, out, aw, s, H_, hd, ws)
    qb, kb, vb = (orc.f32_to_bf16(a)[None] for a in (q, k, v))
    out_ref, aw_ref = orc.swa_forward(qb, kb, vb, ws, H_)
    assert relerr(out, orc.bf16_to_f32(out_ref)[0]) < REL_TOL_BF16
    assert relerr(aw, orc.bf16_to_f32(aw_ref)[0]) < REL_TOL_BF16
    dq, dk, dv = z(s, H_ * hd), z(s, H_ * hd), z(s, H_ * hd)
    aw_f = orc.bf16_to_f32(aw_ref)[0]
    H.swa_backward_dispatch(q, k, v, aw_f, d_out, dq, dk, dv, s, H_, hd, ws)
    rq, rk, rv = orc.swa_backward(qb, kb, vb, aw_ref, d_out[None], ws, H_)
    for got, ref, n in ((dq, rq[0], "d_q"), (dk, rk[0], "d_k"), (dv, rv[0], "d_v")):
        assert relerr(got, ref) < REL_TOL_BF16, n
