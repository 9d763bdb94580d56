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


# ── ErrorBuffer (core/src/conductor.rs:224-261; known answers of its unit tests, :320-381) ──
def _level_like(d):
    sizes = [d * d, d * d, d * d, 2 * d, 1, 2 * d, 1, 2 * d, 1]
    return [zeros(n) for n in sizes]


def test_error_buffer_accumulates_applies_and_resets():
    from nl_hecate_amd.cms import ErrorBuffer
    d = 4
    buf = ErrorBuffer(_level_like(d))
    g1, g2 = _level_like(d), _level_like(d)
    g1[0].fill_(1.0)
    g2[0].fill_(2.0)
    g2[4].fill_(-0.5)   # a bias
    buf.accumulate(g1)
    assert buf.steps_accumulated == 1
    buf.accumulate(g2)
    assert buf.steps_accumulated == 2
    torch.cuda.synchronize()
    assert torch.all(buf.grads[0] == 3.0) and torch.all(buf.grads[4] == -0.5) and not buf.grads[1].any()
    params = _level_like(d)
    params[0].fill_(10.0)
    buf.apply_and_reset(params, 0.1)
    torch.cuda.synchronize()
    assert_close("w_k_mem", host(params[0]), np.full(d * d, 10.0 - 0.1 * 3.0, np.float32), 1e-6)
    assert_close("b_alpha", host(params[4]), np.full(1, 0.05, np.float32), 1e-6)
    assert buf.steps_accumulated == 0 and not any(g.any() for g in buf.grads)
    before = [p.clone() for p in params]
    buf.apply_and_reset(params, 0.1)   # nothing accumulated: parameters untouched (conductor.rs:247)
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(before, params))


def test_error_buffer_health_check():
    from nl_hecate_amd.cms import ErrorBuffer
    d = 4
    buf = ErrorBuffer(_level_like(d))
    g = _level_like(d)
    g[0].fill_(1.0)
    for _ in range(7):
        buf.accumulate(g)
    assert abs(buf.health_check(g) - 7.0) < 1e-5          # conductor.rs:355-373
    assert buf.health_check(_level_like(d)) is None        # :376-381: zero single-step norm
    h = _level_like(d)
    for i, t in enumerate(h):
        t.copy_(torch.from_numpy(rnd(t.numel())))
    buf2 = ErrorBuffer(_level_like(d))
    buf2.accumulate(h)
    buf2.accumulate(g)
    acc = np.sqrt(sum(float(((host(a) + host(b)) ** 2).sum()) for a, b in zip(h, g)))
    single = np.sqrt(sum(float((host(a) ** 2).sum()) for a in h))
    assert abs(buf2.health_check(h) - acc / single) < 1e-5 * acc / single


# ── ContextState (core/src/conductor.rs:156-221) ──
def test_context_state_reset_and_seed_self_ref():
    from nl_hecate_amd.cms import ContextState
    chains, d, k = 6, 8, 2
    mem = [dev(rnd(chains, d, d)) for _ in range(k)]
    mom = [dev(rnd(chains, d, d)) for _ in range(k)]
    sr = [dev(rnd(chains, 6, d, d)), None]
    ptrs = [t.data_ptr() for t in mem + mom + [sr[0]]]
    cs = ContextState(mem, mom, sr)
    inits = [dict(m_k_init=dev(rnd(d, d)), m_v_init=dev(rnd(d, d)), m_q_init=dev(rnd(d, d)), m_eta_init=dev(rnd(d, d)),
                  m_alpha_init=dev(rnd(d, d)), m_mem_init=dev(rnd(d, d))), dict()]
    cs.seed_self_ref(inits)
    torch.cuda.synchronize()
    for c, n in enumerate(("m_k_init", "m_v_init", "m_q_init", "m_eta_init", "m_alpha_init", "m_mem_init")):
        for b in range(chains):
            assert torch.equal(sr[0][b, c], inits[0][n]), (n, b)
    # static projections: only m_mem is seeded, the five projection memories keep their values
    keep = sr[0].clone()
    new_mem = dev(rnd(d, d))
    cs.seed_self_ref([dict(m_mem_init=new_mem)])
    torch.cuda.synchronize()
    assert torch.equal(sr[0][:, :5], keep[:, :5]) and all(torch.equal(sr[0][b, 5], new_mem) for b in range(chains))
    # m_mem_init also lands in the level's carried memory, every chain (conductor.rs:202-204)
    assert all(torch.equal(mem[0][b], new_mem) for b in range(chains))
    cs.reset()
    torch.cuda.synchronize()
    assert not any(t.any() for t in mem + mom) and not sr[0].any()
    assert ptrs == [t.data_ptr() for t in mem + mom + [sr[0]]], "reset is in place"
    # a level without a self-referential block does not stop the walk: [None, adaptive]
    mem2 = [dev(rnd(chains, d, d)) for _ in range(2)]
    sr2 = [None, dev(rnd(chains, 6, d, d))]
    cs2 = ContextState(mem2, None, sr2)
    keep0 = mem2[0].clone()
    cs2.seed_self_ref([dict(), inits[0]])
    torch.cuda.synchronize()
    assert all(torch.equal(sr2[1][b, 0], inits[0]["m_k_init"]) for b in range(chains)), "level 1 is seeded past a static level 0"
    assert torch.equal(mem2[0], keep0)
    # a static-projection level (no block at all) that carries a learned m_mem_init gets its memory seeded
    cs3 = ContextState([dev(rnd(chains, d, d))], None, [None])
    cs3.seed_self_ref([dict(m_mem_init=new_mem)])
    torch.cuda.synchronize()
    assert all(torch.equal(cs3.memory[0][b], new_mem) for b in range(chains))


def test_frozen_read_backward_kernel():
    bs, s, nh, hd = 2, 70, 3, 16
    d, n = nh * hd, 2 * 70
    dy, m = rnd(n, d), rnd(nh, hd, hd)
    dq = zeros(n, d)
    D.call("memory_read_only_backward_f32_rocm", dev(dy), dev(m), dq, n, nh, hd)
    torch.cuda.synchronize()
    want = np.einsum("hij,thi->thj", m.astype(np.float64), dy.reshape(n, nh, hd).astype(np.float64)).reshape(n, d)
    assert_close("d_q", host(dq), want)
