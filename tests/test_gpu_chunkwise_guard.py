"""The chunkwise rule under the reference's production arguments (a finite m_norm_max, an error clip:
cli/configs/gear1_d1024_gpu1.json:14, sfl5_d1024_h100_runpod_v4.json:13-14): the matrix-form kernels serve the
call when a device-side test shows that neither coupling can fire, the sequential kernels otherwise.  Every case
is checked against the oracle's token loop WITH the couplings (oracle/rules.inc, orc.chunkwise_*), and the
kernel timers say which kernels ran."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu
F32_MAX = float(np.finfo(np.float32).max)


def kernels_run(fn):
    """-> names of the instrumented kernels that fn() launched."""
    lib.nlh_kernel_timer_enable(1)
    buf = ctypes.create_string_buffer(8192)
    lib.nlh_kernel_timer_report(buf, len(buf))   # drop what earlier calls left
    fn()
    torch.cuda.synchronize()
    assert lib.nlh_kernel_timer_report(buf, len(buf)) >= 0
    lib.nlh_kernel_timer_enable(0)
    return {item.rsplit(":", 2)[0] for item in buf.value.decode().split(";") if item}


def oracle_pair(x, C, clip, mmax, has_s=True):
    B, s, d = x["k"].shape
    nc = (s + C - 1) // C
    ys, mcs, scs, gs = [], [], [], []
    for b in range(B):
        eta = x["eta"][b] if has_s else None
        y, mc, sc = orc.chunkwise_forward(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], x["theta"][b], eta, x["m0"][b],
                                          x["s0"][b] if has_s else None, C, has_s=has_s, error_clip=clip, m_norm_max=mmax)
        g = orc.chunkwise_backward(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], x["theta"][b], eta, mc,
                                   sc if has_s else None, x["dy"][b], C, has_s=has_s, error_clip=clip, m_norm_max=mmax)
        ys.append(y); mcs.append(mc); scs.append(sc); gs.append(g)
    return np.stack(ys), np.stack(mcs), np.stack(scs), gs


def max_state_norm(x, C):
    """largest |M_t|_F over the sequential trajectory without couplings (what a bound has to sit above or below)"""
    worst, worst_e = 0.0, 0.0
    for b in range(x["k"].shape[0]):
        M, S = x["m0"][b].astype(np.float64), x["s0"][b].astype(np.float64)
        for t in range(x["k"].shape[1]):
            if t % C == 0:
                M0 = M.copy()
            e = M0 @ x["k"][b, t] - x["v"][b, t]
            worst_e = max(worst_e, float(np.linalg.norm(e)))
            S = x["eta"][b, t] * S - x["theta"][b, t] * np.outer(e, x["k"][b, t])
            M = (1 - x["alpha"][b, t]) * M + S
            worst = max(worst, float(np.linalg.norm(M)))
    return worst, worst_e


def run_f32(x, C, clip, mmax):
    B, s, d = x["k"].shape
    nc = (s + C - 1) // C
    t = {n: dev(a) for n, a in x.items()}
    mc, sc, y = zeros(B, nc + 1, d * d), zeros(B, nc + 1, d * d), zeros(B, s, d)
    fwd = lambda: D.call("titans_chunkwise_forward_f32_cuda", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"], t["m0"],
                         t["s0"], mc, sc, y, s, d, B, C, clip, mmax)
    ran_f = kernels_run(fwd)
    g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
    g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
    dm, ds = zeros(d, d), zeros(d, d)
    bwd = lambda: D.call("titans_chunkwise_backward_f32_cuda", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"], mc, sc,
                         t["dy"], g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], dm, ds, s, d, B, C, clip,
                         mmax)
    ran_b = kernels_run(bwd)
    return host(y), host(mc), host(sc), {n: host(a) for n, a in g.items()}, host(dm), ran_f, ran_b


def check(x, C, clip, mmax, got, tol=1e-4):
    y, mc, sc, g, dm = got[:5]
    B, s, d = x["k"].shape
    yo, mco, sco, go = oracle_pair(x, C, clip, mmax)
    assert_close("y", y, yo, tol)
    assert_close("m_chunk_states", mc.reshape(mco.shape), mco, tol)
    for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
        assert_close(n, g[n], np.stack([gi[n] for gi in go]), tol)
    assert_close("d_m_initial", dm, sum(gi["d_m"] for gi in go), tol)


MATRIX = {"cw_local_fwd_kernel", "cw_out_fwd_kernel"}


def test_production_bound_that_never_fires_keeps_the_matrix_form():
    B, s, d, C = 6, 200, 64, 64
    x = rule_inputs(B, s, d, seed=31, m0_scale=0.02)
    worst, worst_e = max_state_norm(x, C)
    assert worst < 50.0
    got = run_f32(x, C, 0.0, 100.0)
    check(x, C, 0.0, 100.0, got)
    ran_f, ran_b = got[5], got[6]
    assert "cw_guard_tracks_kernel" in ran_f and "rule_fwd_kernel" not in ran_f, ran_f   # the forward tests from its own side outputs
    assert "cw_guard_tracks_kernel" in ran_b and not any(n.startswith("rule_bwd") for n in ran_b), ran_b   # test inside the pass
    # and with a clip far above every error, as the reference's sfl5 configuration ships one
    got = run_f32(x, C, 4.0 * worst_e, 100.0)
    check(x, C, 4.0 * worst_e, 100.0, got)
    assert "rule_fwd_kernel" not in got[5], got[5]


def test_bound_that_fires_in_some_chunks_takes_the_sequential_kernels():
    B, s, d, C = 5, 256, 64, 64
    x = rule_inputs(B, s, d, seed=37, m0_scale=0.02)
    worst, _ = max_state_norm(x, C)
    mmax = 0.6 * worst   # reached somewhere, not everywhere
    yo_free, _, _, _ = oracle_pair(x, C, 0.0, F32_MAX)
    yo, _, _, _ = oracle_pair(x, C, 0.0, mmax)
    assert np.abs(yo - yo_free).max() > 1e-3, "the projection must change the result for this case to mean anything"
    got = run_f32(x, C, 0.0, mmax)
    check(x, C, 0.0, mmax, got)
    assert "rule_fwd_kernel" in got[5], got[5]


def test_clip_that_fires_takes_the_sequential_kernels():
    B, s, d, C = 4, 130, 64, 32
    x = rule_inputs(B, s, d, seed=41, m0_scale=0.02)
    _, worst_e = max_state_norm(x, C)
    clip = 0.5 * worst_e
    got = run_f32(x, C, clip, F32_MAX)
    check(x, C, clip, F32_MAX, got)
    assert "rule_fwd_kernel" in got[5], got[5]


def test_backward_alone_after_a_forward_whose_test_fired_and_after_one_whose_test_did_not():
    """The backward picks the order of its work from how the last test came out (stand-alone test first after one that
    fired, test inside the matrix-form pass otherwise); either order gives the reference's numbers, also when the hint
    is wrong for the call: a backward with a bound that fires right after a forward with one that does not, and the
    other way round.  d_m_initial is added to exactly once either way."""
    B, s, d, C = 4, 192, 64, 64
    x = rule_inputs(B, s, d, seed=53, m0_scale=0.02)
    worst, _ = max_state_norm(x, C)
    t = {n: dev(a) for n, a in x.items()}
    nc = (s + C - 1) // C
    for fwd_bound, bwd_bound in ((100.0, 0.6 * worst), (0.6 * worst, 100.0)):
        mc, sc, y = zeros(B, nc + 1, d * d), zeros(B, nc + 1, d * d), zeros(B, s, d)
        D.call("titans_chunkwise_forward_f32_cuda", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"], t["m0"], t["s0"],
               mc, sc, y, s, d, B, C, 0.0, fwd_bound)
        # states of the trajectory the backward's own bound describes
        yo, mco, sco, go = oracle_pair(x, C, 0.0, bwd_bound)
        g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
        g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
        dm, ds = zeros(d, d), zeros(d, d)
        D.call("titans_chunkwise_backward_f32_cuda", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"],
               dev(mco.reshape(B, nc + 1, d * d)), dev(sco.reshape(B, nc + 1, d * d)), t["dy"], g["d_k"], g["d_v"], g["d_q"],
               g["d_alpha"], g["d_theta"], g["d_eta"], dm, ds, s, d, B, C, 0.0, bwd_bound)
        for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
            assert_close(n, host(g[n]), np.stack([gi[n] for gi in go]), 1e-4)
        assert_close("d_m_initial", host(dm), sum(gi["d_m"] for gi in go), 1e-4)


def test_bf16_backward_alone_with_the_hint_wrong_either_way():
    """The same for the bf16 symbols: the matrix-form gradient pass leaves the error and state norms behind and is
    discarded when the test on them fires."""
    B, s, d, C = 4, 192, 64, 64
    x = rule_inputs(B, s, d, seed=59, m0_scale=0.02)
    for n in ("k", "v", "q"):
        x[n] = torch.from_numpy(x[n]).to(torch.bfloat16).to(torch.float32).numpy()
    worst, _ = max_state_norm(x, C)
    t = {n: dev(a) for n, a in x.items()}
    kb, vb, qb = (t[n].to(torch.bfloat16) for n in ("k", "v", "q"))
    nc = (s + C - 1) // C
    for fwd_bound, bwd_bound in ((100.0, 0.6 * worst), (0.6 * worst, 100.0)):
        mc, sc, y = zeros(B, nc + 1, d * d), zeros(B, nc + 1, d * d), zeros(B, s, d)
        D.call("titans_chunkwise_forward_bf16_guarded_rocm", kb, vb, qb, t["alpha"], t["theta"], t["eta"], t["m0"], t["s0"],
               mc, sc, y, s, d, B, C, 0.0, fwd_bound)
        yo, mco, sco, go = oracle_pair(x, C, 0.0, bwd_bound)
        g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
        g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
        dm, ds = zeros(d, d), zeros(d, d)
        ran = kernels_run(lambda: D.call("titans_chunkwise_backward_bf16_guarded_rocm", kb, vb, qb, t["alpha"], t["theta"],
                                         t["eta"], dev(mco.reshape(B, nc + 1, d * d)), dev(sco.reshape(B, nc + 1, d * d)),
                                         t["dy"], g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], dm, ds,
                                         s, d, B, C, 0.0, bwd_bound))
        fires = bwd_bound < worst
        tol = 1e-4 if fires else 1e-2
        for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
            assert_close(n, host(g[n]), np.stack([gi[n] for gi in go]), tol)
        assert_close("d_m_initial", host(dm), sum(gi["d_m"] for gi in go), tol)
        if fires:   # hint said "did not fire": the pass with the test inside ran first and was discarded
            assert "cw_grads_bf16_kernel" in ran and "cw_guard_tracks_kernel" in ran, ran
        else:       # hint said "fired": the stand-alone test ran first and cleared the matrix form
            assert "cw_guard_kernel" in ran and "cw_grads_bf16_kernel" in ran, ran


def test_bound_just_above_the_trajectory_is_still_exact():
    """A bound the triangle-inequality test cannot clear (between the true maximum and the test's estimate) costs the
    sequential kernels but never a wrong result."""
    B, s, d, C = 3, 128, 64, 64
    x = rule_inputs(B, s, d, seed=43, m0_scale=0.02)
    worst, _ = max_state_norm(x, C)
    got = run_f32(x, C, 0.0, 1.05 * worst)
    check(x, C, 0.0, 1.05 * worst, got)


@pytest.mark.parametrize("mmax_scale,expect_matrix", [(None, True), (0.6, False)])
def test_bf16_pair_with_the_production_arguments(mmax_scale, expect_matrix):
    B, s, d, C = 6, 192, 64, 64
    x = rule_inputs(B, s, d, seed=47, m0_scale=0.02)
    bf = lambda a: torch.from_numpy(a).to(torch.bfloat16)
    for n in ("k", "v", "q"):
        x[n] = bf(x[n]).to(torch.float32).numpy()
    worst, _ = max_state_norm(x, C)
    mmax = 100.0 if mmax_scale is None else mmax_scale * worst
    nc = (s + C - 1) // C
    t = {n: dev(a) for n, a in x.items()}
    kb, vb, qb = (t[n].to(torch.bfloat16) for n in ("k", "v", "q"))
    mc, sc, y = zeros(B, nc + 1, d * d), zeros(B, nc + 1, d * d), zeros(B, s, d)
    ran_f = kernels_run(lambda: D.call("titans_chunkwise_forward_bf16_guarded_rocm", kb, vb, qb, t["alpha"], t["theta"], t["eta"],
                                       t["m0"], t["s0"], mc, sc, y, s, d, B, C, 0.0, mmax))
    g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
    g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
    dm, ds = zeros(d, d), zeros(d, d)
    ran_b = kernels_run(lambda: D.call("titans_chunkwise_backward_bf16_guarded_rocm", kb, vb, qb, t["alpha"], t["theta"], t["eta"],
                                       mc, sc, t["dy"], g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
                                       dm, ds, s, d, B, C, 0.0, mmax))
    got = (host(y), host(mc), host(sc), {n: host(a) for n, a in g.items()}, host(dm))
    # bf16 gradient pass: asserted at 1e-2 as for the unguarded pair; the sequential kernels are fp32
    check(x, C, 0.0, mmax, got, tol=1e-2 if expect_matrix else 1e-4)
    assert ("cw_chain_fwd_kernel" in ran_f) and (("rule_fwd_kernel" in ran_f) != expect_matrix), ran_f
    assert ("cw_grads_bf16_kernel" in ran_b) == expect_matrix, ran_b
