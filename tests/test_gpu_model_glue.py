"""GPU parity, through the C ABI, of the kernels around the memory path (LayerNorm, embedding, transpose copy,
cross-entropy, TNT helpers, 1-D pooling, M3 helpers) against the numpy oracle in float32 (relative 1e-4;
copies and gathers bit-exact), including the accumulate (+=) contracts, invalid targets, ragged group sizes and
shapes that are not multiples of the kernels' tiles."""
import ctypes

import numpy as np
import pytest
import torch

from nl_hecate_amd import dispatch as D
from oracle import model_glue as G
from tests.gpu_util import assert_close, dev, host, zeros

pytestmark = pytest.mark.gpu
f32 = np.float32


def _r(seed):
    r = np.random.default_rng(seed)
    return lambda *sh: r.standard_normal(sh).astype(f32)


@pytest.mark.parametrize("n,d", [(37, 96), (1000, 512), (5, 7), (64, 2048)])
def test_layer_norm_forward_backward(n, d):
    rn = _r(n + d)
    x, gamma, beta, go = rn(n, d) * 2 + 0.5, rn(d), rn(d), rn(n, d)
    out, mean, rstd = zeros(n, d), zeros(n), zeros(n)
    D.call("layer_norm_forward_cuda", dev(x), dev(gamma), dev(beta), out, mean, rstd, n, d, 1e-5)
    oo, om, orr = G.layer_norm_forward(x, gamma, beta, 1e-5)
    assert_close("out", host(out), oo)
    assert_close("mean", host(mean), om)
    assert_close("rstd", host(rstd), orr)
    dx = zeros(n, d)
    dg, db = dev(np.full(d, 3.0, f32)), dev(np.full(d, -2.0, f32))   # accumulated into
    D.call("layer_norm_backward_cuda", dev(go), dev(x), dev(gamma), dev(om), dev(orr), dx, dg, db, n, d)
    ox, og, ob = G.layer_norm_backward(go.astype(np.float64), x.astype(np.float64), gamma.astype(np.float64),
                                       om.astype(np.float64), orr.astype(np.float64))
    assert_close("d_x", host(dx), ox)
    assert_close("d_gamma", host(dg) - 3.0, og)
    assert_close("d_beta", host(db) + 2.0, ob)


def test_layer_norm_backward_is_reproducible():
    rn = _r(3)
    n, d = 4096, 512
    x, gamma, go = rn(n, d), rn(d), rn(n, d)
    _, om, orr = G.layer_norm_forward(x, gamma, gamma, 1e-5)
    runs = []
    for _ in range(2):
        dx, dg, db = zeros(n, d), zeros(d), zeros(d)
        D.call("layer_norm_backward_cuda", dev(go), dev(x), dev(gamma), dev(om), dev(orr), dx, dg, db, n, d)
        runs.append((host(dg), host(db)))
    assert np.array_equal(runs[0][0], runs[1][0]) and np.array_equal(runs[0][1], runs[1][1])


@pytest.mark.parametrize("vocab,d,s", [(50, 64, 300), (7, 5, 40), (1000, 512, 2048)])
def test_embedding_gather_scatter_and_transpose(vocab, d, s):
    rn = _r(vocab + s)
    w, g, acc = rn(vocab, d), rn(s, d), rn(vocab, d)
    ids = np.random.default_rng(s).integers(0, vocab, s).astype(np.int32)
    out = zeros(s, d)
    D.call("embedding_gather_cuda", dev(w), dev(ids), out, s, d)
    assert np.array_equal(host(out), G.embedding_gather(w, ids))
    de = dev(acc)
    D.call("embedding_scatter_add_cuda", dev(g), dev(ids), de, s, d)
    assert_close("d_embed", host(de), G.embedding_scatter_add(g.astype(np.float64), ids, acc.astype(np.float64)))
    wt = zeros(d, vocab)
    D.call("transpose_copy_cuda", dev(w), wt, vocab, d)
    assert np.array_equal(host(wt), w.T)


@pytest.mark.parametrize("s,vocab", [(33, 1000), (5, 17), (64, 50257), (1, 1)])
def test_cross_entropy_forward_backward(s, vocab):
    rn = _r(s + vocab)
    logits = 3 * rn(s, vocab)
    targets = np.random.default_rng(vocab).integers(0, vocab, s).astype(np.int32)
    if s > 4:
        targets[1], targets[3] = -1, vocab
    loss = dev(np.full(1, 123.0, f32))   # overwritten, not accumulated (cross_entropy.cu:90)
    D.call("cross_entropy_forward_cuda", dev(logits), dev(targets), loss, s, vocab)
    want = G.cross_entropy_forward(logits.astype(np.float64), targets)
    assert abs(host(loss)[0] - want) <= 1e-4 * max(abs(want), 1.0)
    dl = dev(np.full((s, vocab), 9.0, f32))
    inv = 1.0 / max(int(((targets >= 0) & (targets < vocab)).sum()), 1)
    D.call("cross_entropy_backward_cuda", dev(logits), dev(targets), dl, s, vocab, inv)
    wd = G.cross_entropy_backward(logits.astype(np.float64), targets, inv)
    got = host(dl)
    assert np.abs(got - wd).max() <= 1e-6 * inv + 1e-4 * np.abs(wd).max()
    assert np.all(got[(targets < 0) | (targets >= vocab)] == 0)


def test_tnt_helpers():
    rn = _r(21)
    d, L, N, alpha = 64, 37, 5, 0.95
    m, y, gm = rn(d, d), rn(L, d), rn(d, d)
    md = zeros(N, d * d)
    D.call("tnt_broadcast_m_f32_cuda", dev(m), md, N, d)
    assert np.array_equal(host(md), G.tnt_broadcast_m(m, N))
    ks, vs = zeros(d), zeros(d)
    D.call("tnt_shard_summary_mean_f32_cuda", dev(y), ks, vs, L, d)
    ok, ov = G.tnt_shard_summary_mean(y)
    assert_close("k_sum", host(ks), ok)
    assert np.array_equal(host(ks), host(vs))
    mg = dev(m)
    D.call("tnt_global_update_f32_cuda", mg, dev(ok), dev(ov), d, alpha)
    assert_close("global_m", host(mg), G.tnt_global_update(m, ok, ov, alpha))
    dmo, dk, dv = zeros(d, d), dev(np.ones(d, f32)), dev(np.ones(d, f32))
    D.call("tnt_global_update_backward_f32_cuda", dev(gm), dev(ok), dev(ov), dmo, dk, dv, d, alpha)
    wm, wk, wv = G.tnt_global_update_backward(gm.astype(np.float64), ok.astype(np.float64), ov.astype(np.float64),
                                              alpha, np.ones(d), np.ones(d))
    assert_close("d_m_old", host(dmo), wm)
    assert_close("d_k_sum", host(dk), wk)
    assert_close("d_v_sum", host(dv), wv)
    base = rn(L, d)
    dy = dev(base)
    D.call("tnt_shard_summary_mean_backward_f32_cuda", dev(wk.astype(f32)), dev(wv.astype(f32)), dy, L, d)
    assert_close("d_local_y", host(dy), G.tnt_shard_summary_mean_backward(wk, wv, base.astype(np.float64)))
    a, b, c = rn(1000), rn(1000), zeros(1000)
    D.call("tnt_combine_gradients_f32_cuda", dev(a), dev(b), c, 1000)
    assert np.array_equal(host(c), a + b)


@pytest.mark.parametrize("bs,s,d,C", [(2, 64, 32, 8), (3, 50, 20, 7), (1, 5, 3, 8)])
def test_pooling_pair(bs, s, d, C):
    rn = _r(s + C)
    sf = s // C
    x, go, gu, base = rn(bs, s, d), rn(bs, max(sf, 1), d)[:, :sf], rn(bs, s, d), rn(bs, s, d)
    pooled = zeros(bs, sf, d)
    D.call("mean_pool_1d_f32_cuda", dev(x), pooled, bs, s, d, C)
    op = G.mean_pool_1d(x, C)
    if sf:
        assert_close("pooled", host(pooled), op)
    dx = dev(base)
    D.call("mean_pool_1d_backward_f32_cuda", dev(np.ascontiguousarray(go)), dx, bs, s, d, C)
    assert np.allclose(host(dx), G.mean_pool_1d_backward(np.ascontiguousarray(go), base, C), rtol=1e-6, atol=1e-6)
    up = dev(np.full((bs, s, d), 7.0, f32))
    D.call("repeat_upsample_1d_f32_cuda", dev(op), up, bs, s, d, C)
    assert np.array_equal(host(up), G.repeat_upsample_1d(op, s, C, np.full((bs, s, d), 7.0, f32)))
    dp = zeros(bs, sf, d)
    D.call("repeat_upsample_1d_backward_f32_cuda", dev(gu), dp, bs, s, d, C)
    if sf:
        assert_close("d_pooled", host(dp), G.repeat_upsample_1d_backward(gu.astype(np.float64), C))


def test_m3_helpers():
    rn = _r(8)
    n = 100003
    g, m1, m2, v, w = rn(n), rn(n), rn(n), np.abs(rn(n)), rn(n)
    for upd in (1, 0):
        a, b, c = dev(m1), dev(m2), dev(v)
        assert D.call("m3_ema_update_cuda", a, b, c, dev(g), n, 0.9, 0.99, 0.999, upd) == 0
        o = G.m3_ema_update(m1, m2, v, g, 0.9, 0.99, 0.999, upd)
        for got, want in zip((a, b, c), o):
            assert np.allclose(host(got), want, rtol=1e-6, atol=1e-7)
    wd = dev(w)
    assert D.call("m3_apply_1d_cuda", wd, dev(m1), dev(m2), dev(v), n, 0.01, 0.5, 1e-8, 0.7) == 0
    assert_close("w 1d", host(wd), G.m3_apply_1d(w, m1, m2, v, 0.01, 0.5, 1e-8, 0.7))
    wd = dev(w)
    assert D.call("m3_apply_2d_cuda", wd, dev(m1), dev(m2), n, 0.01, 0.5) == 0
    assert np.allclose(host(wd), G.m3_apply_2d(w, m1, m2, 0.01, 0.5), rtol=1e-6, atol=1e-7)
    xd = dev(w)
    assert D.call("m3_ns_poly_cuda", xd, dev(m1), dev(m2), n, 3.4445, -4.775, 2.0315) == 0
    assert np.allclose(host(xd), G.m3_ns_poly(w, m1, m2, 3.4445, -4.775, 2.0315), rtol=1e-5, atol=1e-6)
    xd = dev(w)
    assert D.call("scale_buf_cuda", xd, 0.25, n) == 0
    assert np.array_equal(host(xd), w * f32(0.25))
    nb = ctypes.c_int(0)
    parts = zeros((n + 255) // 256)
    assert D.call("frob_norm_sq_cuda", dev(w), parts, n, ctypes.byref(nb)) == 0
    assert nb.value == (n + 255) // 256
    assert abs(float(host(parts).astype(np.float64).sum()) - float((w.astype(np.float64) ** 2).sum())) < 1e-4 * n


@pytest.mark.parametrize("s,d,inter", [(37, 48, 100), (512, 512, 1408), (1, 8, 8)])
def test_swiglu_forward_backward(s, d, inter):
    rn = _r(s + inter)
    x, wg, wu, wd, gy = rn(s, d), rn(inter, d) / d ** 0.5, rn(inter, d) / d ** 0.5, rn(d, inter) / inter ** 0.5, rn(s, d)
    y, gate, up, fused, cache = zeros(s, d), zeros(s, inter), zeros(s, inter), zeros(s, inter), zeros(s, inter)
    D.call("swiglu_forward_f32_cuda_dd", dev(x), dev(wg), dev(wu), dev(wd), y, gate, up, fused, cache, s, d, inter)
    x64, g64, u64, d64 = (a.astype(np.float64) for a in (x, wg, wu, wd))
    oy, og, ou, of, osig = G.swiglu_forward(x64, g64, u64, d64)
    for name, got, want in (("y", y, oy), ("gate", gate, og), ("up", up, ou), ("fused", fused, of), ("sigmoid", cache, osig)):
        assert_close(name, host(got), want)
    dx = dev(np.full((s, d), 5.0, f32))   # written fresh, not accumulated
    dg, du, dd = zeros(inter, d), zeros(inter, d), zeros(d, inter)
    D.call("swiglu_backward_f32_cuda_dd", dev(gy), dev(x), dev(wg), dev(wu), dev(wd), fused, gate, up, cache, dx, dg, du,
           dd, s, d, inter)
    wx, wgg, wuu, wdd = G.swiglu_backward(gy.astype(np.float64), x64, g64, u64, d64, of, og, ou, osig)
    for name, got, want in (("d_x", dx, wx), ("d_gate_proj", dg, wgg), ("d_up_proj", du, wuu), ("d_down_proj", dd, wdd)):
        assert_close(name, host(got), want)
