"""Pins oracle/memory_level.py, the CPU composition of one CMS memory level (gpu_memory_forward /
gpu_memory_backward of the reference): its numpy glue against the C oracle's float32 glue, its head layout
against explicit indexing, and its backward against central differences of its own float64 forward."""
import types

import numpy as np
import pytest

from oracle import memory_level as ML
from oracle import pyoracle as orc

F32_MAX = ML.F32_MAX


def cfg_of(rule, nh, hd, **kw):
    base = dict(memory_rule=rule, num_heads=nh, head_dim=hd, checkpoint_interval=None, proxy=False, chunk_size=None,
                alpha_floor=0.0, alpha_ceil=1.0, theta_floor=0.0, theta_ceil=F32_MAX, error_clip=0.0,
                m_norm_max=F32_MAX)
    base.update(kw)
    return types.SimpleNamespace(**base)


def params(d, seed, dt=np.float64):
    r = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: r.uniform(-lim, lim, (d, d)).astype(dt) for n in ("w_k", "w_v", "w_q")}
    for n in ("w_alpha", "w_theta", "w_eta"):
        p[n] = r.uniform(-0.5, 0.5, 2 * d).astype(dt)
    p["b_alpha"], p["b_theta"], p["b_eta"] = (np.array([v], dt) for v in (-1.0, -1.5, 1.0))
    return p


def test_numpy_glue_matches_the_c_oracle():
    r = np.random.default_rng(1)
    f = np.float32
    k, v = r.standard_normal((37, 24)).astype(f), r.standard_normal((37, 24)).astype(f)
    w = r.uniform(-0.3, 0.3, 48).astype(f)
    for act in (0, 1):
        assert np.allclose(ML.gate(k, v, w, np.array([0.2], f), act), orc.gate_compute(k, v, w, 0.2, act), atol=1e-6)
    k[5] = 0.0                      # a row below eps
    xn, norms = ML.l2_normalize(k)
    xo, no = orc.l2_normalize_rows(k)
    assert np.allclose(xn, xo, atol=1e-6) and np.allclose(norms, no, atol=1e-6)
    g = r.standard_normal(k.shape).astype(f)
    # the zero row's gradient is d_out / eps (1e8 times d_out): relative tolerance
    assert np.allclose(ML.l2_normalize_backward(g, xn, norms), orc.l2_normalize_backward(g, xo, no), rtol=1e-5,
                       atol=1e-5)


def test_gate_weight_gradients_match_the_c_oracle():
    r = np.random.default_rng(2)
    f = np.float32
    n, d = 29, 12
    k, v = r.standard_normal((n, d)).astype(f), r.standard_normal((n, d)).astype(f)
    alpha, eta = (r.uniform(0.05, 0.95, n).astype(f) for _ in range(2))
    theta = r.uniform(0.01, 2.0, n).astype(f)
    da, dth, de = (r.standard_normal(n).astype(f) for _ in range(3))
    c = dict(k=k, v=v, q=k, alpha=alpha, theta=theta, eta=eta, k_norms=np.ones(n, f), q_norms=np.ones(n, f))
    p = params(d, 3, f)
    x = r.standard_normal((1, n, d)).astype(f)
    z = np.zeros((n, d), f)
    g, _ = ML.projection_grads(p, x, c, z, z, z, da, dth, de)
    o = orc.gate_backward(da, alpha, dth, theta, de, eta, k, v)
    for name in ("w_alpha", "b_alpha", "w_theta", "b_theta", "w_eta", "b_eta"):
        assert np.allclose(g[name], o["d_" + name], rtol=1e-4, atol=1e-5), name


def test_head_layout():
    bs, s, nh, hd = 2, 5, 3, 4
    x = np.arange(bs * s * nh * hd, dtype=np.float64).reshape(bs * s, nh * hd)
    h = ML.to_heads(x, bs, s, nh, hd)
    for b in range(bs):
        for hh in range(nh):
            for t in range(s):
                assert np.array_equal(h[b * nh + hh, t], x[b * s + t, hh * hd:(hh + 1) * hd])
    assert np.array_equal(ML.from_heads(h, bs, s, nh, hd), x)
    g = np.arange(bs * s, dtype=np.float64)
    gh = ML.gates_to_heads(g, bs, s, nh)
    assert gh.shape == (bs * nh, s) and np.array_equal(gh[1 * nh + 2], g[s:2 * s])
    assert np.array_equal(ML.gates_from_heads(gh, bs, s, nh), nh * g)


VARIANTS = [("delta", {}), ("titans", {}), ("hebbian", {}), ("dgd", {}),
            ("delta", dict(proxy=True, chunk_size=3)), ("titans", dict(proxy=True, chunk_size=4))]


@pytest.mark.parametrize("rule,kw", VARIANTS)
def test_backward_is_the_gradient_of_the_forward(rule, kw):
    """Central differences of L = sum(y * dY) in float64.  The gate weights see the whole forward; the
    projections and the input are differentiated with the gates held at their values, which is the
    gradient the reference computes (accumulate_projection_grads sends nothing from the gates into k, v)."""
    bs, s, nh, hd = 2, 7, 2, 4
    d = nh * hd
    cfg = cfg_of(rule, nh, hd, **kw)
    r = np.random.default_rng(11)
    p = params(d, 5)
    x = r.standard_normal((bs, s, d)) / np.sqrt(d)
    m0 = 0.3 * r.standard_normal((bs * nh, hd, hd))
    dy = r.standard_normal((bs, s, d))
    y, cache, _ = ML.level_forward(p, cfg, x, m0)
    grads, d_x = ML.level_backward(p, cfg, cache, dy, x)
    gates = (cache["alpha"], cache["theta"], cache["eta"])
    eps = 1e-6

    def loss(pp, xx, frozen):
        return float((ML.level_forward(pp, cfg, xx, m0, gates if frozen else None)[0] * dy).sum())

    def fd_param(name, idx, frozen):
        lo, hi = {**p}, {**p}
        lo[name], hi[name] = p[name].copy(), p[name].copy()
        lo[name][idx] -= eps
        hi[name][idx] += eps
        return (loss(hi, x, frozen) - loss(lo, x, frozen)) / (2 * eps)

    names = ["w_alpha", "b_alpha"] + ([] if rule == "hebbian" else ["w_theta", "b_theta"]) \
        + (["w_eta", "b_eta"] if rule == "titans" else [])
    for name in names:
        for idx in ([(0,)] if name[0] == "b" else [(1,), (d + 2,), (2 * d - 1,)]):
            want = fd_param(name, idx, False)
            assert abs(grads[name][idx] - want) <= 1e-6 + 1e-5 * abs(want), (name, idx, grads[name][idx], want)
    for name in ("w_k", "w_v", "w_q"):
        for idx in [(0, 0), (3, 5), (d - 1, 2)]:
            want = fd_param(name, idx, True)
            assert abs(grads[name][idx] - want) <= 1e-6 + 1e-5 * abs(want), (name, idx, grads[name][idx], want)
    for idx in [(0, 0, 0), (1, 3, 5), (0, s - 1, d - 1)]:
        lo, hi = x.copy(), x.copy()
        lo[idx] -= eps
        hi[idx] += eps
        want = (loss(p, hi, True) - loss(p, lo, True)) / (2 * eps)
        assert abs(d_x[idx] - want) <= 1e-6 + 1e-5 * abs(want), (idx, d_x[idx], want)


def test_clamped_gates_pass_no_gradient():
    bs, s, nh, hd = 1, 6, 2, 4
    d = nh * hd
    r = np.random.default_rng(4)
    p = params(d, 6)
    x = r.standard_normal((bs, s, d))
    m0 = np.zeros((bs * nh, hd, hd))
    dy = r.standard_normal((bs, s, d))
    cfg = cfg_of("delta", nh, hd, alpha_floor=0.2, alpha_ceil=0.3, theta_ceil=0.15)
    y, cache, _ = ML.level_forward(p, cfg, x, m0)
    assert cache["alpha"].min() >= 0.2 and cache["alpha"].max() <= 0.3 and cache["theta"].max() <= 0.15
    on_a = (cache["alpha"] <= 0.2) | (cache["alpha"] >= 0.3)
    assert on_a.any()
    grads, _ = ML.level_backward(p, cfg, cache, dy, x)
    if on_a.all():
        assert np.all(grads["w_alpha"] == 0)
    free = cfg_of("delta", nh, hd)
    y2, cache2, _ = ML.level_forward(p, free, x, m0)
    assert np.abs(y - y2).max() > 1e-6


def test_carried_memory_is_clamped():
    bs, s, nh, hd = 1, 5, 1, 4
    r = np.random.default_rng(8)
    p = params(4, 7)
    x = r.standard_normal((bs, s, 4))
    m0 = 2.0 * r.standard_normal((1, 4, 4))
    cfg = cfg_of("hebbian", nh, hd, m_norm_max=0.5)
    _, cache, carried = ML.level_forward(p, cfg, x, m0)
    assert np.sqrt((cache["m_states"][0, -1] ** 2).sum()) > 0.5
    assert abs(np.sqrt((carried[0] ** 2).sum()) - 0.5) < 1e-12


@pytest.mark.parametrize("rule,nh", [("delta", 1), ("titans", 1), ("delta", 3), ("titans", 2)])
def test_tnt_backward_is_the_gradient_of_the_forward(rule, nh):
    """TNT level (shards of local chunks around a global memory), float64: central differences of
    L = sum(y * dY) + sum(M_final * dM) are not needed — the reference's backward starts from a zero gradient of the
    final global memory, so L = sum(y * dY).  Ragged last shard and a padded last local chunk included.
    One head: the reference's attribution of the local chains' initial-memory gradients (all onto head 0) is the
    gradient.  Several heads: it is not; the per-head attribution is, and that is what is checked there."""
    hd, s, cg, cl = 4, 11, 4, 3        # shards of 4, 4, 3 tokens; local chunks of 3 (+ padding)
    d = nh * hd
    cfg = cfg_of(rule, nh, hd)
    r = np.random.default_rng(21)
    p = params(d, 22)
    x = r.standard_normal((s, d)) / np.sqrt(d)
    m0 = 0.3 * r.standard_normal((nh, hd, hd))
    dy = r.standard_normal((s, d))
    y, shards, m_fin = ML.tnt_forward(p, cfg, x, m0, cg, cl)
    assert len(shards) == 3 and shards[0]["padded"] == 6 and shards[2]["padded"] == 3
    grads, d_x = ML.tnt_backward(p, cfg, shards, dy, x, cl, per_head_memory_gradient=nh > 1)
    if nh > 1:   # the reference's attribution differs from the gradient once there is a second head
        ref_grads, _ = ML.tnt_backward(p, cfg, shards, dy, x, cl)
        assert np.abs(ref_grads["w_k"] - grads["w_k"]).max() > 1e-6
    gates = [(c["alpha"], c["theta"], c["eta"]) for c in shards]
    eps = 1e-6

    def loss(pp, xx, frozen):
        return float((ML.tnt_forward(pp, cfg, xx, m0, cg, cl, gates if frozen else None)[0] * dy).sum())

    def fd_param(name, idx, frozen):
        lo, hi = {**p}, {**p}
        lo[name], hi[name] = p[name].copy(), p[name].copy()
        lo[name][idx] -= eps
        hi[name][idx] += eps
        return (loss(hi, x, frozen) - loss(lo, x, frozen)) / (2 * eps)

    names = ["w_alpha", "b_alpha", "w_theta", "b_theta"] + (["w_eta", "b_eta"] if rule == "titans" else [])
    for name in names:
        for idx in ([(0,)] if name[0] == "b" else [(1,), (d + 2,)]):
            want = fd_param(name, idx, False)
            assert abs(grads[name][idx] - want) <= 1e-6 + 1e-5 * abs(want), (name, idx, grads[name][idx], want)
    for name in ("w_k", "w_v", "w_q"):
        for idx in [(0, 0), (3, 1)]:
            want = fd_param(name, idx, True)
            assert abs(grads[name][idx] - want) <= 1e-6 + 1e-5 * abs(want), (name, idx, grads[name][idx], want)
    for idx in [(0, 0), (5, 2), (s - 1, d - 1)]:
        lo, hi = x.copy(), x.copy()
        lo[idx] -= eps
        hi[idx] += eps
        want = (loss(p, hi, True) - loss(p, lo, True)) / (2 * eps)
        assert abs(d_x[idx] - want) <= 1e-6 + 1e-5 * abs(want), (idx, d_x[idx], want)


def test_tnt_with_one_shard_and_one_chunk_is_the_plain_level():
    nh, hd, s = 2, 4, 6
    d = nh * hd
    cfg = cfg_of("titans", nh, hd)
    r = np.random.default_rng(23)
    p = params(d, 24)
    x = r.standard_normal((s, d)) / np.sqrt(d)
    m0 = 0.3 * r.standard_normal((nh, hd, hd))
    y_t, _, _ = ML.tnt_forward(p, cfg, x, m0, s, s)
    y_l, _, _ = ML.level_forward(p, cfg, x[None], m0)
    assert np.allclose(y_t, y_l[0], rtol=1e-12, atol=1e-14)
