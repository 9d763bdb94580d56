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


def _golden_m3():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "m3_known_answers.json")) as f:
        return json.load(f)


def test_m3_moment_updates_match_torch_adam_state_and_the_reference_known_answers():
    """m3_ema_update is Adam's pair of moment updates plus a slow first moment: checked against the state
    torch.optim.Adam keeps (exp_avg, exp_avg_sq) over three steps, and against the known answers of the
    reference's own tests (first step from zero = theta * grad with theta = 1 - eta; constant gradient
    converges to it)."""
    n, b1, b2, b3 = 11, 0.9, 0.99, 0.999
    w = torch.nn.Parameter(torch.zeros(n, dtype=torch.float64))
    opt = torch.optim.Adam([w], lr=1e-3, betas=(b1, b2), eps=1e-8)
    slow = torch.optim.Adam([torch.nn.Parameter(torch.zeros(n, dtype=torch.float64))], lr=1e-3, betas=(b3, b2))
    m1, m2, v = np.zeros(n), np.zeros(n), np.zeros(n)
    for step in range(3):
        g = R.standard_normal(n)
        for o in (opt, slow):
            o.param_groups[0]["params"][0].grad = T(g)
            o.step()
        m1, m2, v = G.m3_ema_update(m1, m2, v, g, b1, b2, b3, True)
        st = opt.state[w]
        assert np.allclose(m1, st["exp_avg"].numpy(), atol=1e-15) and np.allclose(v, st["exp_avg_sq"].numpy(), atol=1e-15)
        assert np.allclose(m2, slow.state[slow.param_groups[0]["params"][0]]["exp_avg"].numpy(), atol=1e-15)
    keep = m2.copy()
    assert np.array_equal(G.m3_ema_update(m1, m2, v, g, b1, b2, b3, False)[1], keep), "update_m2 = 0 leaves the slow moment"
    ka = _golden_m3()
    one = ka["single_step"]
    z = np.zeros(3)
    got = G.m3_ema_update(z, z, z, np.array(one["grad"]), one["eta"], 0.99, 0.999, True)[0]
    assert np.abs(got - np.array(one["update"])).max() < one["abs_tol"]
    cv = ka["ema_convergence"]
    m = np.zeros(1)
    for _ in range(cv["steps"]):
        m = G.m3_ema_update(m, m, m, np.array([cv["grad"]]), cv["eta"], 0.99, 0.999, False)[0]
    assert abs(m[0] - cv["expected"]) < cv["abs_tol"]


def test_m3_parameter_updates_match_torch_adam_and_sgd_steps():
    """m3_apply_1d with alpha = 0 is Adam's parameter update with the first-moment bias correction folded
    into lr (torch: step = lr / bc1 * m / (sqrt(v) / sqrt(bc2) + eps)); the slow moment enters linearly
    (alpha).  m3_apply_2d is a plain gradient step on o1 + alpha o2."""
    n, b1, b2, lr, eps = 9, 0.9, 0.95, 3e-3, 1e-8
    w0 = R.standard_normal(n)
    w = torch.nn.Parameter(T(w0).clone())
    opt = torch.optim.Adam([w], lr=lr, betas=(b1, b2), eps=eps)
    ours, m1, m2, v = w0.copy(), np.zeros(n), np.zeros(n), np.zeros(n)
    for step in range(1, 4):
        g = R.standard_normal(n)
        w.grad = T(g)
        opt.step()
        m1, m2, v = G.m3_ema_update(m1, m2, v, g, b1, b2, 0.999, True)
        ours = G.m3_apply_1d(ours, m1, m2, v, lr / (1 - b1 ** step), 0.0, eps, 1 - b2 ** step)
        assert np.allclose(ours, w.detach().numpy(), atol=1e-13)
    al = 0.37
    assert np.allclose(G.m3_apply_1d(w0, m1, m2, v, lr, al, eps, 0.7), G.m3_apply_1d(w0, m1 + al * m2, 0 * m2, v, lr, 0.0, eps, 0.7),
                       atol=1e-15)
    ws = torch.nn.Parameter(T(w0).clone())
    sgd = torch.optim.SGD([ws], lr=lr)
    ws.grad = T(m1 + al * m2)
    sgd.step()
    assert np.allclose(G.m3_apply_2d(w0, m1, m2, lr, al), ws.detach().numpy(), atol=1e-15)


def _newton_schulz(m, iters, coef):
    """The loop around m3_ns_poly (core/src/gpu_optimizer.rs:975-1000): X <- a X + b (X X^T) X + c (X X^T)^2 X."""
    x = m.copy()
    for _ in range(iters):
        ata = x @ x.T
        ax = ata @ x
        x = G.m3_ns_poly(x, ax, ata @ ax, coef["a"], coef["b"], coef["c"])
    return x


def test_m3_newton_schulz_polynomial():
    """On a scaled orthogonal matrix sigma Q one step must give p(sigma) Q with p(s) = a s + b s^3 + c s^5
    (X X^T = sigma^2 I): a closed form that a swapped or mis-signed coefficient breaks.  Iterated on the
    reference's test matrix the singular values move into the band around 1 the quintic is built for, and
    its known answers hold (finite, non-zero, modified; zero iterations change nothing)."""
    ka = _golden_m3()
    co, ns = ka["coefficients"], ka["newton_schulz"]
    q, _ = np.linalg.qr(R.standard_normal((5, 5)))
    for sigma in (0.3, 0.8, 1.1):
        got = _newton_schulz(sigma * q, 1, co)
        p = co["a"] * sigma + co["b"] * sigma ** 3 + co["c"] * sigma ** 5
        assert np.allclose(got, p * q, atol=1e-12)
    d = ns["d"]
    m = np.array([np.sin(0.37 * i + 0.1) * 0.5 for i in range(d * d)]).reshape(d, d)
    x0 = m / np.linalg.norm(m)
    out = _newton_schulz(x0, ns["iterations"], co)
    assert np.isfinite(out).all() and np.linalg.norm(out) > ns["min_frobenius"] and np.abs(out - m).sum() > ns["min_l1_change"]
    sv = np.linalg.svd(out, compute_uv=False)
    big = np.linalg.svd(x0, compute_uv=False) > 1e-3
    assert np.all((sv[big] > 0.6) & (sv[big] < 1.3)), sv
    z = np.array(ns["zero_iterations_matrix"], float).reshape(3, 3)
    assert np.array_equal(_newton_schulz(z, 0, co), z)


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
