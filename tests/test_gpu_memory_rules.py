"""GPU parity of the exact memory rules (Titans LMM, Delta, DGD) through the
C ABI against the CPU oracle, on the reference's own test recipes and on
config-shaped inputs.  Tolerance: relative 1e-4 (max|a-b|/max|b|) for these
fp32 paths; the reference's absolute 1e-5 / 1e-4 on its own recipes.
"""
import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.ffi import lib
from oracle import pyoracle as orc
from tests.gpu_util import (assert_abs, assert_close, dev, host, rule_inputs, zeros)

pytestmark = pytest.mark.gpu
F32_MAX = orc.F32_MAX


def gpu_titans_forward(x, clip=0.0, mx=F32_MAX, input_stride=None, m_stride=None):
    B, s, d = x["k"].shape
    ms, ss, y = zeros(B, s + 1, d, d), zeros(B, s + 1, d, d), zeros(B, s, d)
    D.titans_forward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                        dev(x["eta"]), dev(x["m0"]), dev(x["s0"]), ms, ss, y, s, d, B,
                        input_stride or s, m_stride or d * d, clip, mx)
    torch.cuda.synchronize()
    return host(y), host(ms), host(ss)


def gpu_delta_forward(x, clip=0.0, mx=F32_MAX, dgd=False):
    B, s, d = x["k"].shape
    ms, y = zeros(B, s + 1, d, d), zeros(B, s, d)
    if dgd:
        D.dgd_forward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                         dev(x["m0"]), ms, y, s, d, B, s, d * d, clip)
    else:
        D.delta_forward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                           dev(x["m0"]), ms, y, s, d, B, s, d * d, clip, mx)
    torch.cuda.synchronize()
    return host(y), host(ms)


def gpu_titans_backward(x, ms, ss, clip=0.0):
    B, s, d = x["k"].shape
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_eta=zeros(B, s), d_m_initial=zeros(d, d), d_s_initial=zeros(d, d))
    D.titans_backward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                         dev(x["eta"]), dev(ms), dev(ss), dev(x["dy"]),
                         g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
                         g["d_m_initial"], g["d_s_initial"], s, d, B, clip)
    torch.cuda.synchronize()
    return {n: host(t) for n, t in g.items()}


def gpu_delta_backward(x, ms, clip=0.0):
    B, s, d = x["k"].shape
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_m_initial=zeros(d, d))
    D.delta_backward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                        dev(ms), dev(x["dy"]), g["d_k"], g["d_v"], g["d_q"], g["d_alpha"],
                        g["d_theta"], g["d_m_initial"], s, d, B, clip)
    torch.cuda.synchronize()
    return {n: host(t) for n, t in g.items()}


def test_lane_primitives_selftest():
    assert lib.nlh_selftest_lane_ops() == 0


# ── the reference's own recipes (core/tests/test_cuda_titans.rs) ───────────
def _ref_recipe(seq_len, d, seeds):
    rb = lambda n, seed: orc.simple_rng_uniform(n, seed, 0.1)
    x = dict(k=rb(seq_len * d, seeds[0]).reshape(1, seq_len, d),
             v=rb(seq_len * d, seeds[1]).reshape(1, seq_len, d),
             q=rb(seq_len * d, seeds[2]).reshape(1, seq_len, d),
             alpha=np.full((1, seq_len), 0.05, np.float32),
             theta=np.full((1, seq_len), 0.01, np.float32),
             eta=np.full((1, seq_len), 0.9, np.float32),
             m0=np.zeros((1, d, d), np.float32), s0=np.zeros((1, d, d), np.float32))
    if len(seeds) > 3:
        x["dy"] = rb(seq_len * d, seeds[3]).reshape(1, seq_len, d)
    return x


def test_titans_forward_reference_recipe():
    """test_cuda_titans.rs:69-97: d=8, s=16, seeds 100/200/300, tol 1e-5 abs."""
    x = _ref_recipe(16, 8, (100, 200, 300))
    y, ms, ss = gpu_titans_forward(x)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    assert_abs("titans_fwd_y", y, yo, 1e-5)
    assert_abs("titans_fwd_m", ms, mo, 1e-5)
    assert_abs("titans_fwd_s", ss, so, 1e-5)
    assert np.abs(ss[0, -1]).max() > 1e-10  # momentum is live (test_cuda_titans.rs:150-155)


def test_titans_forward_seq_len_1():
    """test_cuda_titans.rs:99-128: d=4, s=1, seeds 400/500/600 (the general-head-size kernels)."""
    x = _ref_recipe(1, 4, (400, 500, 600))
    y, ms, ss = gpu_titans_forward(x)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    assert_abs("y", y, yo, 1e-5)
    assert_abs("m", ms, mo, 1e-5)


def test_titans_backward_reference_recipe():
    """test_cuda_titans.rs:160-295: d=8, s=12, seeds 1000..1300, tol 1e-4 abs."""
    x = _ref_recipe(12, 8, (1000, 1100, 1200, 1300))
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    g = gpu_titans_backward(x, mo, so)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"])
    for n in go:
        assert_abs(n, g[n], go[n], 1e-4)
    assert np.abs(g["d_k"]).max() > 0 and np.abs(g["d_eta"]).max() > 0


def test_titans_dispatch_with_clip_and_mnorm_reference_recipe():
    """test_cuda_titans.rs:421-466: clip=1.0, m_norm_max=5.0 through the same entry point."""
    x = rule_inputs(2, 24, 16, 4210, m0_scale=0.5)
    x["v"] *= 4.0  # make the clip bite
    y, ms, ss = gpu_titans_forward(x, 1.0, 5.0)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"], 1.0, 5.0)
    yn, _, _ = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                        x["m0"], x["s0"])
    assert np.abs(yo - yn).max() > 1e-3, "clip/projection must be active in this case"
    assert_close("y", y, yo)
    assert_close("m", ms, mo)
    assert_close("s", ss, so)
    g = gpu_titans_backward(x, mo, so, 1.0)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"], 1.0)
    for n in go:
        assert_close(n, g[n], go[n])


# ── config-shaped inputs over every tiled head dimension ───────────────────
@pytest.mark.parametrize("B,s,d", [(3, 37, 8), (2, 50, 16), (5, 33, 32), (3, 70, 64), (128, 24, 64),
                                   (256, 17, 64), (2, 21, 128)])
def test_titans_forward_backward_parity(B, s, d):
    x = rule_inputs(B, s, d, 1000 + d + B, m0_scale=0.2)
    y, ms, ss = gpu_titans_forward(x)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    assert_close("s_states", ss, so)
    g = gpu_titans_backward(x, mo, so)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"])
    for n in go:
        assert_close(n, g[n], go[n])


@pytest.mark.parametrize("B,s,d", [(4, 64, 64), (3, 19, 16), (130, 20, 64)])
def test_delta_and_dgd_parity(B, s, d):
    x = rule_inputs(B, s, d, 2000 + d + B, m0_scale=0.2)
    y, ms = gpu_delta_forward(x)
    yo, mo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    g = gpu_delta_backward(x, mo)
    go = orc.delta_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], mo, x["dy"])
    for n in go:
        assert_close(n, g[n], go[n])
    # DGD is the Delta rule (core/tests/test_cuda_dgd.rs:521-585): bit-identical here
    yd, md = gpu_delta_forward(x, dgd=True)
    assert np.array_equal(yd, y) and np.array_equal(md, ms)


def test_delta_config1_beta_mapping():
    """BASELINE config 1: Delta, 1 head, d=64, batch 4, seq 512, M0=0; the single
    gate beta maps to theta=beta, alpha=0, and d_beta is d_theta."""
    x = rule_inputs(4, 512, 64, 0x5EED0001)
    x["alpha"][:] = 0
    y, ms = gpu_delta_forward(x)
    yo, mo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"])
    assert_close("y", y, yo)
    g = gpu_delta_backward(x, mo)
    go = orc.delta_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], mo, x["dy"])
    for n in go:
        assert_close(n, g[n], go[n])


@pytest.mark.parametrize("clip,mx", [(0.7, F32_MAX), (0.0, 1.5), (0.7, 1.5)])
@pytest.mark.parametrize("d", [16, 64])
def test_coupled_clip_and_projection(clip, mx, d):
    x = rule_inputs(3, 29, d, 3000 + d, m0_scale=0.3)
    x["v"] *= 2.0
    y, ms, ss = gpu_titans_forward(x, clip, mx)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"], clip, mx)
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    if mx < 1e30:
        assert np.sqrt((ms[:, 1:] ** 2).sum((2, 3))).max() <= mx * (1 + 1e-5)
    g = gpu_titans_backward(x, mo, so, clip)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   mo, so, x["dy"], clip)
    for n in go:
        assert_close(n, g[n], go[n])
    yd, md = gpu_delta_forward(x, clip, mx)
    ydo, mdo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"], clip, mx)
    assert_close("delta y", yd, ydo)


def test_forward_stride_contract():
    """Segment replay calls the forward with input_stride = full seq_len and
    m_stride = n_ckpt*dd (core/src/gpu_backward.rs:1924-1939)."""
    B, s, d = 3, 40, 64
    x = rule_inputs(B, s, d, 4000, m0_scale=0.2)
    t0, seg = 16, 11
    n_slots = 3
    m_init = np.zeros((B, n_slots, d, d), np.float32)
    s_init = np.zeros((B, n_slots, d, d), np.float32)
    m_init[:, 1] = x["m0"]
    s_init[:, 1] = x["s0"]
    ms, ss, y = zeros(B, seg + 1, d, d), zeros(B, seg + 1, d, d), zeros(B, seg, d)
    k, v, q = dev(x["k"]), dev(x["v"]), dev(x["q"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    mi, si = dev(m_init), dev(s_init)
    D.titans_forward_dd(k.view(-1)[t0 * d:], v.view(-1)[t0 * d:], q.view(-1)[t0 * d:],
                        al.view(-1)[t0:], th.view(-1)[t0:], et.view(-1)[t0:],
                        mi.view(-1)[d * d:], si.view(-1)[d * d:], ms, ss, y,
                        seg, d, B, s, n_slots * d * d, 0.0, F32_MAX)
    torch.cuda.synchronize()
    sl = slice(t0, t0 + seg)
    yo, mo, so = orc.titans_forward_batch(x["k"][:, sl], x["v"][:, sl], x["q"][:, sl],
                                          x["alpha"][:, sl], x["theta"][:, sl], x["eta"][:, sl],
                                          x["m0"], x["s0"])
    assert_close("y", host(y), yo)
    assert_close("m", host(ms), mo)
    assert_close("s", host(ss), so)


# ── checkpointed forward + segment backward (the reference's schedule) ─────
@pytest.mark.parametrize("C", [1, 4, 8, 64, 5])
def test_checkpointed_schedule_equals_full(C):
    """core/tests/test_gradient_checkpoint.rs:140-280 with the orchestration of
    core/src/gpu_backward.rs:1876-1962 (replay forward, then segment backward)."""
    B, s, d = 3, 19, 64
    x = rule_inputs(B, s, d, 5000 + C, m0_scale=0.2)
    n = orc.checkpoint_count(s, C)
    k, v, q, dy = dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["dy"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    mc, sc, y = zeros(B, n, d, d), zeros(B, n, d, d), zeros(B, s, d)
    D.call("titans_forward_ckpt_batched_f32_rocm", k, v, q, al, th, et, dev(x["m0"]), dev(x["s0"]),
           mc, sc, y, s, d, B, C, 0.0, F32_MAX)
    yf, mf, sf = gpu_titans_forward(x)
    slots = [0] + [t + 1 for t in range(s) if (t + 1) % C == 0 or t + 1 == s]
    assert np.array_equal(host(y), yf), "checkpointed forward == full forward, bit for bit"
    assert np.array_equal(host(mc), mf[:, slots]) and np.array_equal(host(sc), sf[:, slots])
    # single-chain reference entry point agrees with the batched one
    mc1, sc1, y1 = zeros(n, d, d), zeros(n, d, d), zeros(s, d)
    D.titans_forward_dd_ckpt(k[1], v[1], q[1], al[1], th[1], et[1], dev(x["m0"][1]), dev(x["s0"][1]),
                             mc1, sc1, y1, s, d, C, 0.0, F32_MAX)
    assert np.array_equal(host(mc1), host(mc)[1]) and np.array_equal(host(y1), yf[1])

    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_eta=zeros(B, s))
    seed_m, seed_s = zeros(B, d, d), zeros(B, d, d)
    max_seg = min(C, s)
    lm, ls, ly = zeros(B, max_seg + 1, d, d), zeros(B, max_seg + 1, d, d), zeros(B, max_seg, d)
    segs = [(t, min(t + C, s), i) for i, t in enumerate(range(0, s, C))]
    for t0, t1, ci in reversed(segs):
        seg = t1 - t0
        D.titans_forward_dd(k.view(-1)[t0 * d:], v.view(-1)[t0 * d:], q.view(-1)[t0 * d:],
                            al.view(-1)[t0:], th.view(-1)[t0:], et.view(-1)[t0:],
                            mc.view(-1)[ci * d * d:], sc.view(-1)[ci * d * d:], lm, ls, ly,
                            seg, d, B, s, n * d * d, 0.0, F32_MAX)
        out_m, out_s = zeros(B, d, d), zeros(B, d, d)
        D.titans_backward_dd_segment(k, v, q, al, th, et, lm, ls, dy, seed_m, seed_s,
                                     g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"],
                                     g["d_eta"], out_m, out_s, t0, t1, d, B, s, 0.0)
        seed_m, seed_s = out_m, out_s
    torch.cuda.synchronize()
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                   *orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"],
                                                             x["theta"], x["eta"], x["m0"], x["s0"])[1:],
                                   x["dy"])
    for nme in g:
        assert_close(nme, host(g[nme]), go[nme])
    assert_close("d_m_initial", host(seed_m).sum(0), go["d_m_initial"])
    assert_close("d_s_initial", host(seed_s).sum(0), go["d_s_initial"])


def test_backward_accumulates_initial_state_grads_and_is_deterministic():
    B, s, d = 6, 33, 64
    x = rule_inputs(B, s, d, 6000, m0_scale=0.2)
    _, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                         x["m0"], x["s0"])
    g1 = gpu_titans_backward(x, mo, so)
    g2 = gpu_titans_backward(x, mo, so)
    for n in g1:
        assert np.array_equal(g1[n], g2[n]), f"{n} differs between identical runs"
    # accumulate contract: a second call adds onto the caller's buffer
    acc = torch.full((d, d), 1.0, dtype=torch.float32, device="cuda")
    junk = [zeros(B, s, d) for _ in range(3)] + [zeros(B, s) for _ in range(3)]
    D.titans_backward_dd(dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["alpha"]), dev(x["theta"]),
                         dev(x["eta"]), dev(mo), dev(so), dev(x["dy"]), *junk, acc, zeros(d, d),
                         s, d, B, 0.0)
    torch.cuda.synchronize()
    assert_close("accumulated", host(acc) - 1.0, g1["d_m_initial"], 1e-4)


def test_argument_errors_are_reported():
    lib.nlh_set_error_mode(1)
    try:
        lib.nlh_clear_error()
        z = zeros(8)
        D.call("titans_forward_f32_cuda", z, z, z, z, z, z, z, z, z, z, z, 4, 0, 1, 4, 0, 0.0, 0.0)
        assert b"d=0" in lib.nlh_last_error()
        lib.nlh_clear_error()
        # refused before any launch: the per-token vectors of this head size do not fit in LDS
        D.call("titans_forward_f32_cuda", z, z, z, z, z, z, z, z, z, z, z, 4, 20000, 1, 4, 0, 0.0, 0.0)
        assert b"beyond the general kernels" in lib.nlh_last_error()
        lib.nlh_clear_error()
        D.call("titans_forward_ckpt_f32_cuda", z, z, z, z, z, z, z, z, z, z, z, 4, 8, 0, 0.0, 0.0)
        assert b"checkpoint_interval" in lib.nlh_last_error()
    finally:
        lib.nlh_clear_error()
        lib.nlh_set_error_mode(0)


# ── one-call checkpointed backward: fused (on-chip replay) and replay schedule ──
def _oracle_ckpt_grads(x, C, has_s, clip=0.0, mx=F32_MAX):
    B, s, d = x["k"].shape
    outs = []
    for b in range(B):
        y, mc, sc = orc.forward_ckpt(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], x["theta"][b],
                                     x["eta"][b], x["m0"][b], x["s0"][b], C, has_s, clip, mx)
        outs.append(orc.backward_ckpt(x["k"][b], x["v"][b], x["q"][b], x["alpha"][b], x["theta"][b],
                                      x["eta"][b], mc, sc, x["dy"][b], C, has_s, clip, mx))
    g = {n: np.stack([o[n] for o in outs]) for n in outs[0] if n not in ("d_m", "d_s")}
    g["d_m_initial"] = sum(o["d_m"] for o in outs)
    g["d_s_initial"] = sum(o["d_s"] for o in outs)
    return g


def _gpu_ckpt_fwd_bwd(x, C, has_s, entry, clip=0.0, mx=F32_MAX):
    B, s, d = x["k"].shape
    n = orc.checkpoint_count(s, C)
    k, v, q, dy = dev(x["k"]), dev(x["v"]), dev(x["q"]), dev(x["dy"])
    al, th, et = dev(x["alpha"]), dev(x["theta"]), dev(x["eta"])
    mc, sc, y = zeros(B, n, d, d), zeros(B, n, d, d), zeros(B, s, d)
    g = dict(d_k=zeros(B, s, d), d_v=zeros(B, s, d), d_q=zeros(B, s, d), d_alpha=zeros(B, s),
             d_theta=zeros(B, s), d_m_initial=zeros(d, d))
    if has_s:
        g.update(d_eta=zeros(B, s), d_s_initial=zeros(d, d))
        D.call("titans_forward_ckpt_batched_f32_rocm", k, v, q, al, th, et, dev(x["m0"]), dev(x["s0"]),
               mc, sc, y, s, d, B, C, clip, mx)
        D.call("titans_backward_ckpt" + entry + "_f32_rocm", k, v, q, al, th, et, mc, sc, dy,
               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_eta"],
               g["d_m_initial"], g["d_s_initial"], s, d, B, C, clip, mx)
    else:
        D.call("delta_forward_ckpt_batched_f32_rocm", k, v, q, al, th, dev(x["m0"]), mc, y,
               s, d, B, C, clip, mx)
        D.call("delta_backward_ckpt" + entry + "_f32_rocm", k, v, q, al, th, mc, dy,
               g["d_k"], g["d_v"], g["d_q"], g["d_alpha"], g["d_theta"], g["d_m_initial"],
               s, d, B, C, clip, mx)
    torch.cuda.synchronize()
    return {n_: host(t) for n_, t in g.items()}


@pytest.mark.parametrize("entry", ["", "_replay"])
@pytest.mark.parametrize("B,s,d,C", [(3, 200, 64, 64), (2, 19, 64, 5), (2, 77, 64, 64), (3, 50, 16, 8),
                                     (2, 40, 32, 16), (2, 30, 128, 64), (1, 130, 8, 64),
                                     (2, 150, 64, 100), (2, 9, 64, 1), (5, 64, 64, 64)])
def test_checkpointed_backward_one_call(entry, B, s, d, C):
    x = rule_inputs(B, s, d, 7000 + s + d + C, m0_scale=0.2)
    for has_s in (True, False):
        g = _gpu_ckpt_fwd_bwd(x, C, has_s, entry)
        go = _oracle_ckpt_grads(x, C, has_s)
        for n in g:
            assert_close(f"{n} has_s={has_s}", g[n], go[n])


def _saturate(x, s, C):
    """alpha exactly 0 and 1 (retention 1 and 0), eta exactly 0 and 1, theta 0: at segment edges, inside
    segments, at the first and the last token, and in runs."""
    spots = {0: (0.0, 1.0, None), 3: (1.0, 0.0, None), C - 1: (1.0, 1.0, 0.0), C: (0.0, 0.0, None),
             C + 7: (1.0, None, None), 2 * C: (None, 0.0, 0.0), s - 1: (1.0, 1.0, None)}
    for t, (a, e, th) in spots.items():
        if a is not None: x["alpha"][:, t] = a
        if e is not None: x["eta"][:, t] = e
        if th is not None: x["theta"][:, t] = th
    x["alpha"][1, 10:20] = 0.0
    x["eta"][1, C + 10:C + 20] = 1.0
    return x


@pytest.mark.parametrize("d", [16, 64])
def test_saturated_gates_full_trajectory(d):
    B, s = 2, 70
    x = _saturate(rule_inputs(B, s, d, 7300 + d, m0_scale=0.2), s, 32)
    y, ms, ss = gpu_titans_forward(x)
    yo, mo, so = orc.titans_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"],
                                          x["m0"], x["s0"])
    assert_close("y", y, yo)
    assert_close("m_states", ms, mo)
    assert_close("s_states", ss, so)
    g = gpu_titans_backward(x, mo, so)
    go = orc.titans_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["eta"], mo, so, x["dy"])
    for n in go:
        assert np.isfinite(g[n]).all(), n
        assert_close(n, g[n], go[n])
    yd, md = gpu_delta_forward(x)
    ydo, mdo = orc.delta_forward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], x["m0"])
    assert_close("delta y", yd, ydo)
    gd = gpu_delta_backward(x, mdo)
    gdo = orc.delta_backward_batch(x["k"], x["v"], x["q"], x["alpha"], x["theta"], mdo, x["dy"])
    for n in gdo:
        assert_close("delta " + n, gd[n], gdo[n])


@pytest.mark.parametrize("entry", ["", "_replay"])
@pytest.mark.parametrize("d,C", [(64, 64), (16, 8)])
def test_saturated_gates_checkpointed(entry, d, C):
    B, s = 2, 3 * C + 5
    x = _saturate(rule_inputs(B, s, d, 7400 + d, m0_scale=0.2), s, C)
    for has_s in (True, False):
        g = _gpu_ckpt_fwd_bwd(x, C, has_s, entry)
        go = _oracle_ckpt_grads(x, C, has_s)
        for n in g:
            assert np.isfinite(g[n]).all(), n
            assert_close(f"{n} has_s={has_s}", g[n], go[n])


def test_checkpointed_backward_with_clip_takes_replay_schedule():
    x = rule_inputs(2, 40, 64, 7100, m0_scale=0.3)
    x["v"] *= 2.0
    g = _gpu_ckpt_fwd_bwd(x, 16, True, "", clip=0.7, mx=1.5)
    go = _oracle_ckpt_grads(x, 16, True, 0.7, 1.5)
    for n in g:
        assert_close(n, g[n], go[n])


def test_checkpointed_backward_is_deterministic():
    x = rule_inputs(4, 130, 64, 7200, m0_scale=0.2)
    g1 = _gpu_ckpt_fwd_bwd(x, 64, True, "")
    g2 = _gpu_ckpt_fwd_bwd(x, 64, True, "")
    for n in g1:
        assert np.array_equal(g1[n], g2[n]), n
