"""Checkpointed backward of the exact Titans / Delta rule in chunk-parallel matrix form (csrc/exact_mm.hip; the rule of
core/kernels/titans_backward.cu:66-341 run from the checkpoints of core/src/gpu_backward.rs:1770-1962).  Every case
goes through the reference-named entry points and is checked against the oracle's token loops; the kernel timers say
that the matrix-form kernels served the call."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, rule_inputs, zeros

pytestmark = pytest.mark.gpu


def kernels_run(fn):
    lib.nlh_kernel_timer_enable(1)
    buf = ctypes.create_string_buffer(8192)
    lib.nlh_kernel_timer_report(buf, len(buf))
    fn()
    torch.cuda.synchronize()
    assert lib.nlh_kernel_timer_report(buf, len(buf)) >= 0
    lib.nlh_kernel_timer_enable(0)
    return {item.rsplit(":", 2)[0] for item in buf.value.decode().split(";") if item}


def oracle_pair(x, C, mmax=None, clip=0.0):
    kw = {} if mmax is None else {"m_norm_max": mmax}
    if clip:
        kw["error_clip"] = clip
    B = x["k"].shape[0]
    cks, gs = [], []
    for b in range(B):
        a = [x[n][b] for n in ("k", "v", "q", "alpha", "theta", "eta")]
        _, mco, sco = orc.forward_ckpt(*a, x["m0"][b], x["s0"][b], C, **kw)
        gs.append(orc.backward_ckpt(*a, mco, sco, x["dy"][b], C, **kw))
        cks.append((mco, sco))
    return cks, gs


def gpu_backward(x, cks, C, mmax, clip=0.0, poison=False):
    B, s, d = x["k"].shape
    t = {n: dev(a) for n, a in x.items()}
    mc = dev(np.stack([c[0] for c in cks]).reshape(B, -1, d * d))
    sc = dev(np.stack([c[1] for c in cks]).reshape(B, -1, d * d))
    mk = (lambda *sh: torch.full(sh, 7.5, dtype=torch.float32, device="cuda")) if poison else zeros
    g = {n: mk(B, s, d) for n in ("d_k", "d_v", "d_q")}
    g.update({n: mk(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
    dm, ds = zeros(d, d), zeros(d, d)
    ran = kernels_run(lambda: D.call("titans_backward_ckpt_f32_rocm", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"],
                                     mc, sc, t["dy"], g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
                                     dm, ds, s, d, B, C, clip, mmax))
    return {n: host(a) for n, a in g.items()}, host(dm), host(ds), ran


def check(got, gs, tol=1e-4):
    g, dm, ds = got[:3]
    for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta", "d_eta"):
        assert_close(n, g[n], np.stack([gi[n] for gi in gs]), tol)
    assert_close("d_m_initial", dm, sum(gi["d_m"] for gi in gs), tol)
    assert_close("d_s_initial", ds, sum(gi["d_s"] for gi in gs), tol)


F32_MAX = float(np.finfo(np.float32).max)


@pytest.fixture(autouse=True)
def matrix_form_wherever_it_applies():
    """The library picks the form by a cost model (short test sequences would go to the sequential kernel)."""
    prev = lib.nlh_exact_backward_form(1)
    yield
    lib.nlh_exact_backward_form(prev)


@pytest.mark.parametrize("B,s,C", [(3, 128, 64), (5, 200, 64), (2, 64, 64), (4, 100, 32), (1, 330, 48), (7, 65, 64), (2, 40, 64)])
def test_titans_against_the_token_loops(B, s, C):
    x = rule_inputs(B, s, 64, seed=101 + s, m0_scale=0.02)
    cks, gs = oracle_pair(x, C)
    got = gpu_backward(x, cks, C, F32_MAX, poison=True)
    check(got, gs)
    assert {"ex_local_kernel", "ex_scan_kernel", "ex_grads_kernel"} <= got[3], got[3]


@pytest.mark.parametrize("B,s,C", [(2, 1, 64), (3, 5, 64), (2, 129, 1), (3, 64, 7), (1, 97, 16), (9, 63, 63), (2, 130, 33)])
def test_edge_shapes(B, s, C):
    """One-token sequences and chunks, intervals that divide nothing, a last chunk of one token."""
    x = rule_inputs(B, s, 64, seed=211 + 7 * s + C, m0_scale=0.02)
    cks, gs = oracle_pair(x, C)
    got = gpu_backward(x, cks, C, F32_MAX, poison=True)
    check(got, gs)
    assert "ex_grads_kernel" in got[3], got[3]


def test_twice_the_upstream_gradient_gives_twice_the_gradients_at_full_size():
    """BASELINE configs[1] at full size (64 chains x 2048 tokens, checkpoints every 64): the backward is linear in d_y
    (the values themselves are checked against the oracle in test_gpu_fullsize_values.py)."""
    B, s, d, C = 64, 2048, 64, 64
    x = rule_inputs(B, s, d, seed=223, m0_scale=0.02)
    t = {n: dev(a) for n, a in x.items()}
    n_ck = orc.checkpoint_count(s, C)
    mc, sc, y = zeros(B, n_ck, d * d), zeros(B, n_ck, d * d), zeros(B, s, d)
    D.call("titans_forward_ckpt_batched_f32_rocm", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"], t["m0"], t["s0"],
           mc, sc, y, s, d, B, C, 0.0, F32_MAX)
    outs = []
    for scale in (1.0, 2.0):
        g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
        g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta", "d_eta")})
        dm, ds = zeros(d, d), zeros(d, d)
        D.call("titans_backward_ckpt_f32_rocm", t["k"], t["v"], t["q"], t["alpha"], t["theta"], t["eta"], mc, sc,
               t["dy"] * scale, g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"], dm, ds, s, d, B, C, 0.0,
               F32_MAX)
        outs.append({**g, "d_m": dm, "d_s": ds})
    for n in outs[0]:
        assert_close(n, host(outs[1][n]), 2.0 * host(outs[0][n]), 1e-5)


def test_saturated_gates():
    """theta = 0, alpha in {0, 1}, eta in {0, 1} on some tokens: nothing divides by a gate."""
    B, s, C = 3, 160, 64
    x = rule_inputs(B, s, 64, seed=113, m0_scale=0.02)
    rng = np.random.default_rng(5)
    for n, vals in (("theta", (0.0,)), ("alpha", (0.0, 1.0)), ("eta", (0.0, 1.0))):
        m = rng.random((B, s)) < 0.15
        x[n][m] = rng.choice(vals, size=int(m.sum())).astype(np.float32)
    cks, gs = oracle_pair(x, C)
    got = gpu_backward(x, cks, C, F32_MAX)
    check(got, gs)
    assert "ex_grads_kernel" in got[3]


def test_delta_rule():
    B, s, d, C = 4, 150, 64, 64
    x = rule_inputs(B, s, d, seed=127, m0_scale=0.02)
    t = {n: dev(a) for n, a in x.items()}
    cks, gs = [], []
    for b in range(B):
        a = [x[n][b] for n in ("k", "v", "q", "alpha", "theta")]
        _, mco, _ = orc.forward_ckpt(*a, None, x["m0"][b], None, C, has_s=False)
        gs.append(orc.backward_ckpt(*a, None, mco, None, x["dy"][b], C, has_s=False))
        cks.append(mco)
    mc = dev(np.stack(cks).reshape(B, -1, d * d))
    g = {n: zeros(B, s, d) for n in ("d_k", "d_v", "d_q")}
    g.update({n: zeros(B, s) for n in ("d_alpha", "d_theta")})
    dm = zeros(d, d)
    ran = kernels_run(lambda: D.call("delta_backward_ckpt_f32_rocm", t["k"], t["v"], t["q"], t["alpha"], t["theta"], mc, t["dy"],
                                     g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], dm, s, d, B, C, 0.0, F32_MAX))
    for n in ("d_k", "d_v", "d_q", "d_alpha", "d_theta"):
        assert_close(n, host(g[n]), np.stack([gi[n] for gi in gs]), 1e-4)
    assert_close("d_m_initial", host(dm), sum(gi["d_m"] for gi in gs), 1e-4)
    assert "ex_grads_kernel" in ran, ran


def worst_norm(x):
    worst, werr = 0.0, 0.0
    for b in range(x["k"].shape[0]):
        M, S = x["m0"][b].astype(np.float64), x["s0"][b].astype(np.float64)
        for t in range(x["k"].shape[1]):
            e = M @ x["k"][b, t] - x["v"][b, t]
            werr = max(werr, float(np.linalg.norm(e)))
            S = x["eta"][b, t] * S - x["theta"][b, t] * np.outer(e, x["k"][b, t])
            M = (1 - x["alpha"][b, t]) * M + S
            worst = max(worst, float(np.linalg.norm(M)))
    return worst, werr


def test_bound_never_reached_keeps_the_matrix_form_and_one_that_fires_leaves_it():
    """m_norm_max = 100 as the reference's configurations ship it (cli/configs/gear1_d1024_gpu1.json:14): the matrix form
    serves the call behind the device-side test; a bound inside the trajectory sends the call to the kernels that
    project, with the initial-state gradients added exactly once; the call after that starts with those kernels and
    returns to the matrix form once a test has passed again."""
    B, s, C = 4, 192, 64
    x = rule_inputs(B, s, 64, seed=131, m0_scale=0.02)
    worst, _ = worst_norm(x)
    cks, gs = oracle_pair(x, C, 100.0)
    # whatever ran before in this process may have left "the last test fired" behind: a first call clears it (its own
    # test, of either form, passes)
    check(gpu_backward(x, cks, C, 100.0), gs)
    got = gpu_backward(x, cks, C, 100.0)
    check(got, gs)
    assert "ex_grads_kernel" in got[3] and "cw_guard_tracks_kernel" in got[3], got[3]
    small = 0.6 * worst
    cks2, gs2 = oracle_pair(x, C, small)
    got2 = gpu_backward(x, cks2, C, small)
    check(got2, gs2)
    assert "ex_grads_kernel" in got2[3] and "rule_fwd_kernel" in got2[3], sorted(got2[3])   # discarded, then the replay schedule
    got3 = gpu_backward(x, cks2, C, small)
    check(got3, gs2)
    assert "ex_grads_kernel" not in got3[3], got3[3]
    got4 = gpu_backward(x, cks, C, 100.0)     # the sequential kernels' own test passes: the hint is cleared
    check(got4, gs)
    got5 = gpu_backward(x, cks, C, 100.0)
    check(got5, gs)
    assert "ex_grads_kernel" in got5[3], got5[3]


def test_error_clip_that_never_fires_and_one_that_does():
    B, s, C = 3, 128, 64
    x = rule_inputs(B, s, 64, seed=137, m0_scale=0.02)
    _, werr = worst_norm(x)
    cks, gs = oracle_pair(x, C, None, clip=2.0 * werr)
    got = gpu_backward(x, cks, C, F32_MAX, clip=2.0 * werr)
    check(got, gs)
    assert "ex_grads_kernel" in got[3], got[3]
    cks2, gs2 = oracle_pair(x, C, None, clip=0.5 * werr)
    got2 = gpu_backward(x, cks2, C, F32_MAX, clip=0.5 * werr)
    check(got2, gs2)
    got3 = gpu_backward(x, cks, C, F32_MAX, clip=2.0 * werr)   # one call goes to the sequential kernels directly
    check(got3, gs)
    assert "ex_grads_kernel" not in got3[3], got3[3]
    got4 = gpu_backward(x, cks, C, F32_MAX, clip=2.0 * werr)
    check(got4, gs)
    assert "ex_grads_kernel" in got4[3], got4[3]


def test_cost_model_picks_the_form():
    """Default setting: one long chain goes to the matrix form (the sequential kernel would leave the chip idle),
    many 8-token chains stay on the sequential kernel; both match the token loops."""
    lib.nlh_exact_backward_form(0)
    x = rule_inputs(1, 1024, 64, seed=149, m0_scale=0.02)
    cks, gs = oracle_pair(x, 64)
    got = gpu_backward(x, cks, 64, F32_MAX)
    check(got, gs)
    assert "ex_grads_kernel" in got[3], got[3]
    x = rule_inputs(300, 8, 64, seed=151, m0_scale=0.02)
    cks, gs = oracle_pair(x, 8)
    got = gpu_backward(x, cks, 8, F32_MAX)
    check(got, gs)
    assert "ex_grads_kernel" not in got[3] and "rule_bwd_fused_kernel" in got[3], got[3]
