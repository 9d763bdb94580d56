"""GPU tests of the CMS dispatch pieces: frequency-aware AdamW under scripted
pulses (per-level step counters, core/src/adamw.rs:437-500), the level
combine + MAG gate and its backward, the frozen-level read."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from nl_hecate_amd.cms import Conductor, FrequencyAwareAdamW
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
R = np.random.default_rng(21)
rnd = lambda *s: R.standard_normal(s).astype(np.float32)


def test_frequency_aware_adamw_under_scripted_pulses():
    k, cs = 3, [1, 2, 4]
    b1, b2, eps, wd, lr, mx = 0.9, 0.95, 1e-8, 0.1, 1e-2, 1.0
    groups = [-1, -1, 0, 0, 1, 2, 2]
    sizes = [700, 3, 1024, 1, 513, 64, 2]
    W = [rnd(n) for n in sizes]
    M = [np.zeros(n, np.float32) for n in sizes]
    V = [np.zeros(n, np.float32) for n in sizes]
    dW, dM, dV = [dev(a) for a in W], [dev(a) for a in M], [dev(a) for a in V]
    dG = [zeros(n) for n in sizes]
    opt = FrequencyAwareAdamW(k, b1, b2, eps, wd)
    ids = [opt.add_tensor(g, w, gr, m, v) for g, w, gr, m, v in zip(groups, dW, dG, dM, dV)]
    opt.set_clamp(ids[3], -10.0, 2.0)  # the level-0 bias stand-in for b_theta
    W[3][:] = 1.999
    dW[3].copy_(torch.from_numpy(W[3]))
    cond = Conductor(k, cs)
    ns = zeros(2)
    swa_step, lvl_step = 0, [0] * k
    for it in range(9):
        pulse = cond.pulse()
        G = [rnd(n) * (5.0 if it % 2 else 0.01) for n in sizes]
        G[3][:] = -50.0  # pushes the clamped bias upward
        for t, g in zip(dG, G):
            t.copy_(torch.from_numpy(g))
        opt.step(pulse, lr, mx, ns)
        torch.cuda.synchronize()
        norm, scale = orc.grad_norm_clip(G, mx)
        assert_close("norm", host(ns)[0], norm, 1e-5)
        assert_close("scale", host(ns)[1], scale, 1e-5)
        swa_step += 1
        for l in range(k):
            lvl_step[l] += int(pulse.active_levels[l])
        for i, g in enumerate(groups):
            if g >= 0 and not pulse.active_levels[g]:
                continue
            t = swa_step if g < 0 else lvl_step[g]
            orc.adamw_step(W[i], G[i] * np.float32(scale), M[i], V[i], lr, b1, b2, eps,
                           1 / (1 - b1 ** t), 1 / (1 - b2 ** t), wd)
        W[3] = np.clip(W[3], -10.0, 2.0) if pulse.active_levels[0] else W[3]
        for i in range(len(sizes)):
            assert_close(f"w[{i}] step {it}", host(dW[i]), W[i], 2e-5)
            assert_close(f"m[{i}] step {it}", host(dM[i]), M[i], 2e-5)
        cond.advance()
    assert opt.swa_step() == 9
    assert [opt.level_step(l) for l in range(k)] == [9, 5, 3] == lvl_step
    assert host(dW[3]).max() <= 2.0


@pytest.mark.parametrize("k", [1, 2, 4])
def test_combine_gate_and_backward(k):
    n = 5003
    ys = [rnd(n) for _ in range(k)]
    attn = rnd(n)
    dys = [dev(y) for y in ys]
    ptrs = (ctypes.c_void_p * k)(*[t.data_ptr() for t in dys])
    yc, gate, gated = zeros(n), zeros(n), zeros(n)
    D.call("cms_combine_gate_rocm", ptrs, k, dev(attn), yc, gate, gated, n)
    c = 1 / np.sqrt(k) if k > 2 else 1.0
    want_yc = np.sum(ys, 0, dtype=np.float64) * c
    want_gate = 1 / (1 + np.exp(-want_yc))
    assert_close("y_comb", host(yc), want_yc, 1e-5)
    assert_close("gate", host(gate), want_gate, 1e-5)
    assert_close("gated", host(gated), attn * want_gate, 1e-5)
    dg = rnd(n)
    d_attn, d_y = zeros(n), zeros(n)
    D.call("cms_gate_backward_rocm", dev(dg), dev(attn), gate, k, d_attn, d_y, n)
    assert_close("d_attn", host(d_attn), dg * want_gate, 1e-5)
    assert_close("d_y", host(d_y), dg * attn * want_gate * (1 - want_gate) * c, 1e-5)


def test_frozen_level_read_only():
    n_tok, nh, hd = 133, 4, 64
    q = rnd(n_tok, nh * hd)
    m = rnd(nh, hd, hd) * 0.1
    y = zeros(n_tok, nh * hd)
    D.call("memory_read_only_f32_rocm", dev(q), dev(m), y, n_tok, nh, hd)
    want = np.einsum("hij,thj->thi", m.astype(np.float64), q.reshape(n_tok, nh, hd)).reshape(n_tok, nh * hd)
    assert_close("y", host(y), want, 1e-5)
