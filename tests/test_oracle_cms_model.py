"""Pins oracle/cms_model.py, the CPU composition of the reference's whole training step (gpu_cms_forward /
gpu_cms_backward): its float attention against the oracle's bf16 attention, and its backward against central
differences of its float64 forward (all levels active: a frozen level passes no gradient in the reference's
path, which no finite difference reproduces; gates held fixed for everything upstream of them, as in
tests/test_oracle_memory_level.py)."""
import types

import numpy as np
import pytest

from oracle import cms_model as CM
from oracle import pyoracle as orc
from tests.test_oracle_memory_level import cfg_of, params

f64 = np.float64


def model(d, v, k, seed, dt=f64, residual=False):
    r = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: r.uniform(-lim, lim, (d, d)).astype(dt) for n in ("w_q", "w_k", "w_v", "w_o")}
    p["w_embed"] = (r.standard_normal((v, d)) / np.sqrt(d) * 2).astype(dt)
    p["w_unembed"] = (r.standard_normal((d, v)) / np.sqrt(d)).astype(dt)
    p["levels"] = [params(d, seed + 10 + i, dt) for i in range(k)]
    if residual:
        for n in ("ln_attn_gamma", "ln_mem_gamma"):
            p[n] = (1.0 + 0.1 * r.standard_normal(d)).astype(dt)
        for n in ("ln_attn_beta", "ln_mem_beta"):
            p[n] = (0.1 * r.standard_normal(d)).astype(dt)
    return p


def config(rule, k, nh, hd, v, s, window, n_p=0, residual=False, parallel=None, **kw):
    return types.SimpleNamespace(d_model=nh * hd, vocab_size=v, num_heads=nh, head_dim=hd, window_size=window, seq_len=s,
                                 n_persistent=n_p, residual=residual, parallel=parallel,
                                 levels=[cfg_of(rule, nh, hd, **kw) for _ in range(k)])


def test_float_attention_matches_the_bf16_oracle():
    r = np.random.default_rng(0)
    s, nh, hd, window, n_p = 19, 2, 8, 5, 2
    bits = [orc.f32_to_bf16(r.standard_normal((1, s, nh * hd)).astype(np.float32)) for _ in range(3)]
    out, aw = orc.swa_forward(*bits, window, nh, n_p)
    q, k, v = (orc.bf16_to_f32(b)[0].astype(f64) for b in bits)
    o, w = CM.swa_float_forward(q, k, v, window, nh, n_p)
    assert np.abs(o - orc.bf16_to_f32(out)[0]).max() < 2e-2 * np.abs(o).max()
    mask = CM.swa_mask(s, window, n_p)
    assert np.all(w[:, ~mask] == 0) and np.allclose(w.sum(-1), 1.0)
    assert mask[10].sum() == window + n_p and mask[10, :n_p].all() and mask[10, 6:11].all() and not mask[10, 2:6].any()
    # its backward against central differences
    go = r.standard_normal((s, nh * hd))
    dq, dk, dv = CM.swa_float_backward(q, k, v, w, go, nh)
    eps = 1e-6
    for arr, grad, idx in ((q, dq, (7, 3)), (k, dk, (1, 9)), (v, dv, (12, 0))):
        hi, lo = arr.copy(), arr.copy()
        hi[idx] += eps
        lo[idx] -= eps
        args = lambda a: [a if t is arr else t for t in (q, k, v)]
        fd = ((CM.swa_float_forward(*args(hi), window, nh, n_p)[0] - CM.swa_float_forward(*args(lo), window, nh, n_p)[0])
              * go).sum() / (2 * eps)
        assert abs(grad[idx] - fd) < 1e-6 + 1e-6 * abs(fd)


CASES = [("delta", 1, False, None, 1), ("titans", 3, False, None, 2), ("titans", 2, True, None, 1),
         ("delta", 2, False, types.SimpleNamespace(tnt_global_chunk_size=4, tnt_local_chunk_size=2), 1)]


@pytest.mark.parametrize("rule,k,residual,parallel,bs", CASES)
def test_backward_is_the_gradient_of_the_forward(rule, k, residual, parallel, bs):
    nh, hd, v, s, window = (1 if parallel else 2), 4, 13, 7, 3
    d = nh * hd
    cfg = config(rule, k, nh, hd, v, s, window, n_p=1, residual=residual, parallel=parallel)
    p = model(d, v, k, 80 + k, residual=residual)
    r = np.random.default_rng(3)
    ids = r.integers(0, v, bs * s)
    tgt = r.integers(0, v, bs * s)
    tgt[2] = -1                                   # an ignored position
    mem = [0.2 * r.standard_normal((bs * nh, hd, hd)) for _ in range(k)]
    active = [True] * k
    loss, c, _ = CM.forward(p, cfg, ids, tgt, active, mem, quantize=False)
    g = CM.backward(p, cfg, c)
    gates = []
    for lc in c["level_caches"]:
        gates.append([(sh["alpha"], sh["theta"], sh["eta"]) for sh in lc] if isinstance(lc, list)
                     else (lc["alpha"], lc["theta"], lc["eta"]))
    eps = 1e-6

    def fd(get, frozen):
        vals = []
        for sign in (+1, -1):
            pp = {n: (a.copy() if isinstance(a, np.ndarray) else [dict((m, b.copy()) for m, b in l.items()) for l in a])
                  for n, a in p.items()}
            get(pp)[...] += sign * eps
            vals.append(CM.forward(pp, cfg, ids, tgt, active, mem, quantize=False, gates=gates if frozen else None)[0])
        return (vals[0] - vals[1]) / (2 * eps)

    checks = [("w_embed", (int(ids[1]), 2)), ("w_q", (1, 3)), ("w_k", (0, 0)), ("w_v", (3, 1)), ("w_o", (2, 2)),
              ("w_unembed", (1, 5))]
    if residual:
        checks += [("ln_attn_gamma", (1,)), ("ln_attn_beta", (0,)), ("ln_mem_gamma", (3,)), ("ln_mem_beta", (2,))]
    view = lambda a, idx: a[idx[0]:idx[0] + 1] if len(idx) == 1 else a[idx[0]:idx[0] + 1, idx[1]:idx[1] + 1]
    for name, idx in checks:
        want = fd(lambda pp: view(pp[name], idx), True)
        assert abs(g[name][idx] - want) <= 1e-7 + 2e-5 * abs(want), (name, idx, g[name][idx], want)
    for lv in range(k):
        for name, idx, frozen in (("w_k", (1, 2), True), ("w_v", (0, 3), True), ("w_q", (2, 0), True),
                                  ("w_alpha", (3,), False), ("b_theta", (0,), False)):
            want = fd(lambda pp: view(pp["levels"][lv][name], idx), frozen)
            got = g["levels"][lv][name][idx]
            assert abs(got - want) <= 1e-7 + 2e-5 * abs(want), (lv, name, idx, got, want)


def test_loss_counts_valid_targets_only():
    nh, hd, v, s = 1, 4, 9, 5
    cfg = config("delta", 1, nh, hd, v, s, 3)
    p = model(4, v, 1, 5)
    ids = np.arange(s) % v
    mem = [np.zeros((1, 4, 4))]
    l_all, _, _ = CM.forward(p, cfg, ids, np.array([1, 2, 3, 4, 5]), [True], mem, quantize=False)
    l_some, c, _ = CM.forward(p, cfg, ids, np.array([1, -1, 3, 99, 5]), [True], mem, quantize=False)
    rows = -np.log(np.exp(c["logits"] - c["logits"].max(1, keepdims=True)) /
                   np.exp(c["logits"] - c["logits"].max(1, keepdims=True)).sum(1, keepdims=True))
    assert abs(l_some - (rows[0, 1] + rows[2, 3] + rows[4, 5]) / 3) < 1e-12 and l_all != l_some
    assert CM.forward(p, cfg, ids, np.full(s, -1), [True], mem, quantize=False)[0] == 0.0
