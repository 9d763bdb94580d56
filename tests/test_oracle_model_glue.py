"""Pins the numpy oracle of the kernels around the memory path (oracle/model_glue.py) against library
routines that are not restatements of it: torch's layer_norm / cross_entropy / avg_pool1d /
repeat_interleave / embedding in float64 with autograd for every backward, and closed forms.  CPU only."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import model_glue as G

R = np.random.default_rng(11)
T = lambda a, grad=False: torch.tensor(a, dtype=torch.float64, requires_grad=grad)


def test_layer_norm_matches_torch_and_autograd():
    n, d, eps = 7, 12, 1e-5
    x, gamma, beta, go = R.standard_normal((n, d)), R.standard_normal(d), R.standard_normal(d), R.standard_normal((n, d))
    out, mean, rstd = G.layer_norm_forward(x, gamma, beta, eps)
    xt, gt, bt = T(x, True), T(gamma, True), T(beta, True)
    ot = F.layer_norm(xt, (d,), gt, bt, eps)
    assert np.allclose(out, ot.detach().numpy(), atol=1e-12)
    assert np.allclose(mean, x.mean(1), atol=1e-13) and np.allclose(rstd, 1 / np.sqrt(x.var(1) + eps), atol=1e-12)
    ot.backward(T(go))
    dx, dg, db = G.layer_norm_backward(go, x, gamma, mean, rstd)
    assert np.allclose(dx, xt.grad.numpy(), atol=1e-11)
    assert np.allclose(dg, gt.grad.numpy(), atol=1e-11) and np.allclose(db, bt.grad.numpy(), atol=1e-12)


def test_cross_entropy_matches_torch_with_ignored_targets():
    s, vocab = 9, 17
    logits = 3 * R.standard_normal((s, vocab))
    targets = R.integers(0, vocab, s).astype(np.int32)
    targets[2], targets[5] = -1, vocab   # both kinds of invalid target are skipped
    valid = (targets >= 0) & (targets < vocab)
    lt = T(logits, True)
    tt = torch.tensor(np.where(valid, targets, -100), dtype=torch.long)
    loss = F.cross_entropy(lt, tt, ignore_index=-100, reduction="sum")
    assert abs(G.cross_entropy_forward(logits, targets) - loss.item()) < 1e-11
    inv = 1.0 / valid.sum()
    (loss * inv).backward()
    d = G.cross_entropy_backward(logits, targets, inv)
    assert np.allclose(d, lt.grad.numpy(), atol=1e-13)
    assert np.all(d[~valid] == 0) and np.allclose(d[valid].sum(1), 0, atol=1e-14)


def test_embedding_transpose_and_scatter():
    vocab, d, s = 11, 5, 20
    w = R.standard_normal((vocab, d))
    ids = R.integers(0, vocab, s).astype(np.int32)
    assert np.array_equal(G.embedding_gather(w, ids), F.embedding(torch.tensor(ids, dtype=torch.long), T(w)).numpy())
    g, acc = R.standard_normal((s, d)), R.standard_normal((vocab, d))
    want = acc.copy()
    np.add.at(want, ids, g)
    assert np.allclose(G.embedding_scatter_add(g, ids, acc), want, atol=1e-14)
    m = R.standard_normal((3, 7))
    assert np.array_equal(G.transpose_copy(m), m.T) and G.transpose_copy(m).flags["C_CONTIGUOUS"]


def test_tnt_helpers_against_autograd():
    d, L, alpha = 6, 5, 0.9
    y, m = R.standard_normal((L, d)), R.standard_normal((d, d))
    ks, vs = G.tnt_shard_summary_mean(y)
    assert np.allclose(ks, y.mean(0)) and np.array_equal(ks, vs)
    assert np.array_equal(G.tnt_broadcast_m(m, 3), np.stack([m.ravel()] * 3))
    mt, kt, vt = T(m, True), T(ks, True), T(vs, True)
    new = alpha * mt + torch.outer(vt, kt)
    assert np.allclose(G.tnt_global_update(m, ks, vs, alpha), new.detach().numpy(), atol=1e-14)
    gm = R.standard_normal((d, d))
    new.backward(T(gm))
    z = np.zeros(d)
    dm, dk, dv = G.tnt_global_update_backward(gm, ks, vs, alpha, z, z)
    assert np.allclose(dm, mt.grad.numpy()) and np.allclose(dk, kt.grad.numpy()) and np.allclose(dv, vt.grad.numpy())
    # mean-pool backward: both summaries are the same mean, so their gradients add
    yt = T(y, True)
    (yt.mean(0) * T(dk)).sum().backward()
    (yt.mean(0) * T(dv)).sum().backward()
    base = R.standard_normal((L, d))
    assert np.allclose(G.tnt_shard_summary_mean_backward(dk, dv, base) - base, yt.grad.numpy(), atol=1e-14)


def test_pooling_pair_against_torch(C=3):
    bs, s, d = 2, 11, 4    # 11 = 3 full groups + 2 tokens that take no part
    sf = s // C
    x = R.standard_normal((bs, s, d))
    pooled = G.mean_pool_1d(x, C)
    assert np.allclose(pooled, F.avg_pool1d(T(x).transpose(1, 2), C).transpose(1, 2).numpy(), atol=1e-14)
    xt = T(x, True)
    go = R.standard_normal((bs, sf, d))
    (F.avg_pool1d(xt.transpose(1, 2), C).transpose(1, 2) * T(go)).sum().backward()
    base = R.standard_normal((bs, s, d))
    assert np.allclose(G.mean_pool_1d_backward(go, base, C) - base, xt.grad.numpy(), atol=1e-14)
    canary = np.full((bs, s, d), 7.0)
    up = G.repeat_upsample_1d(pooled, s, C, canary)
    assert np.array_equal(up[:, :sf * C], torch.repeat_interleave(T(pooled), C, dim=1).numpy())
    assert np.all(up[:, sf * C:] == 7.0)
    pt = T(pooled, True)
    gu = R.standard_normal((bs, s, d))
    (torch.repeat_interleave(pt, C, dim=1) * T(gu[:, :sf * C])).sum().backward()
    assert np.allclose(G.repeat_upsample_1d_backward(gu, C), pt.grad.numpy(), atol=1e-14)


def test_m3_helpers_closed_forms():
    n = 8
    g, m1, m2, v, w = (R.standard_normal(n) for _ in range(5))
    v = np.abs(v)
    a, b, c = G.m3_ema_update(m1, m2, v, g, 0.9, 0.99, 0.999, True)
    assert np.allclose(a, 0.9 * m1 + 0.1 * g) and np.allclose(c, 0.99 * v + 0.01 * g * g)
    assert np.allclose(b, 0.999 * m2 + 0.001 * g)
    assert np.array_equal(G.m3_ema_update(m1, m2, v, g, 0.9, 0.99, 0.999, False)[1], m2)
    assert np.allclose(G.m3_apply_1d(w, m1, m2, v, 0.1, 0.5, 1e-8, 0.7), w - 0.1 * (m1 + 0.5 * m2) / (np.sqrt(v / 0.7) + 1e-8))
    assert np.allclose(G.m3_apply_2d(w, m1, m2, 0.1, 0.5), w - 0.1 * (m1 + 0.5 * m2))
    assert np.allclose(G.m3_ns_poly(w, m1, m2, 3.4445, -4.775, 2.0315), 3.4445 * w - 4.775 * m1 + 2.0315 * m2)


def test_swiglu_matches_torch_silu_mlp_and_autograd():
    s, d, inter = 6, 5, 9
    x, wg, wu, wd, gy = (R.standard_normal(sh) for sh in ((s, d), (inter, d), (inter, d), (d, inter), (s, d)))
    y, gate, up, fused, sig = G.swiglu_forward(x, wg, wu, wd)
    xt, gt, ut, dt = T(x, True), T(wg, True), T(wu, True), T(wd, True)
    yt = (F.silu(xt @ gt.T) * (xt @ ut.T)) @ dt.T
    assert np.allclose(y, yt.detach().numpy(), atol=1e-12)
    yt.backward(T(gy))
    dx, dg, du, dd = G.swiglu_backward(gy, x, wg, wu, wd, fused, gate, up, sig)
    for got, want in ((dx, xt.grad), (dg, gt.grad), (du, ut.grad), (dd, dt.grad)):
        assert np.allclose(got, want.numpy(), atol=1e-11)
