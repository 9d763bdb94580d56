"""GPU parity of the per-level memory step on device buffers (nl_hecate_amd.memory_level: the host mirror of the
reference's gpu_memory_forward / gpu_memory_backward and its GpuMemoryCache variants) against the CPU
composition of the same step from the oracle's rules (oracle/memory_level.py), float32, relative 1e-4 unless
stated.  Every variant: outputs, cached tensors, the carried memory, parameter gradients and d_embedded."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import memory_level as GL
from nl_hecate_amd.mag_layer import MemoryLevelParams
from oracle import memory_level as ML
from oracle import pyoracle as orc
from tests.gpu_util import assert_close, dev, host

pytestmark = pytest.mark.gpu

NAMES = ("w_k", "w_v", "w_q", "w_alpha", "b_alpha", "w_theta", "b_theta", "w_eta", "b_eta")


def params(d, seed):
    r = np.random.default_rng(seed)
    lim = np.sqrt(6.0 / (2 * d))
    p = {n: r.uniform(-lim, lim, (d, d)).astype(np.float32) for n in ("w_k", "w_v", "w_q")}
    for n in ("w_alpha", "w_theta", "w_eta"):
        p[n] = r.uniform(-0.5, 0.5, 2 * d).astype(np.float32)
    p["b_alpha"], p["b_theta"], p["b_eta"] = (np.array([v], np.float32) for v in (-1.0, -1.5, 1.0))
    return p


def run_both(cfg, bs, s, seed, m0_scale=0.3):
    nh, hd = cfg.num_heads, cfg.head_dim
    d = nh * hd
    r = np.random.default_rng(seed)
    p = params(d, seed + 1)
    x = (r.standard_normal((bs, s, d)) / np.sqrt(d)).astype(np.float32)
    m0 = (m0_scale * r.standard_normal((bs * nh, hd, hd))).astype(np.float32)
    dy = r.standard_normal((bs, s, d)).astype(np.float32)
    y_o, c_o, carried_o = ML.level_forward(p, cfg, x, m0)
    g_o, dx_o = ML.level_backward(p, cfg, c_o, dy, x)
    lp = MemoryLevelParams(*[dev(p[n]) for n in NAMES])
    ctx = dev(m0.reshape(bs * nh, hd * hd))
    emb = dev(x.reshape(bs * s, d))
    y, cache = GL.gpu_memory_forward(lp, cfg, emb, ctx, s, d, bs)
    grads = GL.LevelGrads.zeros(d)
    d_emb = GL.gpu_memory_backward(lp, cfg, cache, dev(dy.reshape(bs * s, d)), emb, grads, s, d, bs)
    torch.cuda.synchronize()
    return dict(y=(host(y).reshape(bs, s, d), y_o), cache=(cache, c_o), carried=(host(ctx), carried_o),
                grads=(grads, g_o), d_x=(host(d_emb).reshape(bs, s, d), dx_o), B=bs * nh, hd=hd)


def check(out, kind, tol=1e-4, has_theta=True, has_eta=False):
    cache, c_o = out["cache"]
    assert cache.kind == kind
    assert_close("y", *out["y"], tol)
    for n, on in (("k_mem", "k"), ("v_mem", "v"), ("q_mem", "q"), ("alpha", "alpha"), ("k_norms", "k_norms"),
                  ("q_norms", "q_norms")):
        assert_close(n, host(getattr(cache, n)).reshape(c_o[on].shape), c_o[on], tol)
    if has_theta:
        assert_close("theta", host(cache.theta), c_o["theta"], tol)
    else:
        assert cache.theta is None
    if has_eta:
        assert_close("eta", host(cache.eta), c_o["eta"], tol)
        assert_close("s_states", host(cache.s_states).reshape(c_o["s_states"].shape), c_o["s_states"], tol)
    else:
        assert cache.eta is None and cache.s_states is None
    assert_close("m_states", host(cache.m_states).reshape(c_o["m_states"].shape), c_o["m_states"], tol)
    assert_close("carried", out["carried"][0].reshape(out["carried"][1].shape), out["carried"][1], tol)
    grads, g_o = out["grads"]
    for n in ("w_k", "w_v", "w_q"):
        assert_close("d_" + n, host(getattr(grads, f"d_{n}_mem")), g_o[n], tol)
    gate_names = ["alpha"] + (["theta"] if has_theta else []) + (["eta"] if has_eta else [])
    for n in gate_names:
        assert_close("d_w_" + n, host(getattr(grads, "d_w_" + n)), g_o["w_" + n], tol)
        assert_close("d_b_" + n, host(getattr(grads, "d_b_" + n)), g_o["b_" + n], tol)
    assert_close("d_embedded", *out["d_x"], tol)


FULL = [("delta", "Delta", True, False), ("titans", "Titans", True, True), ("hebbian", "Hebbian", False, False),
        ("dgd", "DGD", True, False)]


@pytest.mark.parametrize("rule,kind,has_theta,has_eta", FULL)
@pytest.mark.parametrize("bs,s,nh,hd", [(1, 24, 2, 8), (2, 17, 3, 16), (1, 9, 1, 32)])
def test_full_trajectory_variants(rule, kind, has_theta, has_eta, bs, s, nh, hd):
    cfg = GL.LevelConfig(rule, nh, hd)
    check(run_both(cfg, bs, s, 100 + s + hd), kind, has_theta=has_theta, has_eta=has_eta)


@pytest.mark.parametrize("rule,kind,has_theta,has_eta", [
    ("delta", "DeltaCkpt", True, False), ("titans", "TitansCkpt", True, True),
    ("hebbian", "HebbianCkpt", False, False), ("dgd", "DGDCkpt", True, False)])
@pytest.mark.parametrize("bs,s,nh,hd,C", [(1, 24, 2, 8, 8), (1, 22, 2, 16, 8), (2, 13, 2, 8, 4), (1, 6, 1, 16, 16)])
def test_checkpointed_variants(rule, kind, has_theta, has_eta, bs, s, nh, hd, C):
    """Batch sizes above 1 go beyond the reference, which refuses them for the checkpointed variants."""
    cfg = GL.LevelConfig(rule, nh, hd, checkpoint_interval=C)
    out = run_both(cfg, bs, s, 200 + s + C)
    assert out["cache"][0].m_states.shape[1] == GL.checkpoint_count(s, C)
    check(out, kind, has_theta=has_theta, has_eta=has_eta)


@pytest.mark.parametrize("rule,kind,has_eta", [("delta", "DeltaChunkwise", False), ("titans", "TitansChunkwise", True)])
@pytest.mark.parametrize("bs,s,nh,hd,cs", [(1, 24, 2, 8, 8), (2, 21, 2, 16, 4), (1, 10, 1, 8, None), (1, 12, 2, 8, 1)])
def test_chunkwise_variants(rule, kind, has_eta, bs, s, nh, hd, cs):
    cfg = GL.LevelConfig(rule, nh, hd, proxy=True, chunk_size=cs)
    out = run_both(cfg, bs, s, 300 + s)
    c = out["cache"][0]
    assert c.chunk_size == (cs or s) and c.num_chunks == -(-s // (cs or s))
    check(out, kind, has_eta=has_eta)


@pytest.mark.parametrize("rule,kind,has_eta", [("delta", "Delta", False), ("titans", "Titans", True)])
def test_gate_clamps_error_clip_and_norm_bound(rule, kind, has_eta):
    """CS-39 clamps with their straight-through masks, the error clip and the per-token / carried norm bound."""
    cfg = GL.LevelConfig(rule, 2, 8, alpha_floor=0.22, alpha_ceil=0.3, theta_floor=0.05, theta_ceil=0.2,
                         error_clip=0.7, m_norm_max=1.5)
    out = run_both(cfg, 2, 20, 77, m0_scale=0.6)
    c = out["cache"][0]
    a, th = host(c.alpha), host(c.theta)
    assert a.min() >= 0.22 - 1e-7 and a.max() <= 0.3 + 1e-7 and th.max() <= 0.2 + 1e-7
    assert (a == np.float32(0.22)).any() or (a == np.float32(0.3)).any()
    carried = out["carried"][0].reshape(-1, 64)
    assert np.sqrt((carried ** 2).sum(-1)).max() <= 1.5 * (1 + 1e-5)
    check(out, kind, tol=2e-4, has_eta=has_eta)


def test_gate_statistics_and_delta_norm():
    v = np.random.default_rng(3).uniform(0.0, 1.0, 1001).astype(np.float32)
    st = GL.GateStats.from_slice(v, 0.1, True)
    assert st.count == 1001 and st.min == v.min() and st.max == v.max()
    assert abs(st.median - np.quantile(v.astype(np.float64), 0.5)) < 1e-6
    assert abs(st.p95 - np.quantile(v.astype(np.float64), 0.95)) < 1e-6
    assert abs(st.p99 - np.quantile(v.astype(np.float64), 0.99)) < 1e-6
    assert st.frac_at_bound == float((v <= np.float32(0.1 * (1 + 1e-4))).sum()) / 1001
    assert GL.GateStats.from_slice(v, 0.0, True).frac_at_bound == 0.0
    assert GL.GateStats.from_slice(v, 0.9, False).frac_at_bound == float((v >= np.float32(0.9 * (1 - 1e-4))).sum()) / 1001
    assert GL.GateStats.from_slice(v, GL.F32_MAX, False).frac_at_bound == 0.0
    # |M_{s-1} k_{s-1} - v_{s-1}| from the cached trajectory, one head, batch 1
    cfg = GL.LevelConfig("delta", 1, 16)
    out = run_both(cfg, 1, 11, 5)
    cache, c_o = out["cache"]
    want = np.linalg.norm(c_o["m_states"][0, 10] @ c_o["k"][10] - c_o["v"][10])
    assert abs(cache.dgd_delta_norm(11, 16, 1, 1) - want) <= 1e-4 * want
    assert cache.alpha_stats(0.0).count == 11 and cache.eta_stats() is None
    assert abs(cache.theta_stats(GL.F32_MAX).mean - c_o["theta"].mean()) < 1e-5
    cfg = GL.LevelConfig("titans", 1, 16, proxy=True, chunk_size=4)
    out = run_both(cfg, 1, 11, 6)
    cache, c_o = out["cache"]
    want = np.linalg.norm(c_o["m_states"][0, 2] @ c_o["k"][10] - c_o["v"][10])   # start of the last chunk
    assert abs(cache.dgd_delta_norm(11, 16, 1, 1) - want) <= 1e-4 * want
    assert cache.eta_stats().count == 11
    assert GL.LevelConfig("hebbian", 2, 8) and out["cache"][0].dgd_delta_norm(11, 16, 1, 2) == 0.0


@pytest.mark.parametrize("act", ["gelu", "silu", "relu"])
@pytest.mark.parametrize("bs,s,nh,hd,factor", [(1, 6, 2, 8, 4), (2, 9, 1, 8, 3)])
def test_titans_with_an_mlp_memory(act, bs, s, nh, hd, factor):
    """memory_layers = 2: the packed {W1, b1, W2, b2} state per head (gpu_forward.rs:1473-1510)."""
    cfg = GL.LevelConfig("titans", nh, hd, memory_layers=2, memory_expansion_factor=factor, memory_activation=act)
    d, dh = nh * hd, factor * hd
    n_state = orc.mlp_state_size(hd, dh)
    r = np.random.default_rng(31 + s)
    p = params(d, 32)
    x = (r.standard_normal((bs, s, d)) / np.sqrt(d)).astype(np.float32)
    m0 = (0.3 * r.standard_normal((bs * nh, n_state)) / np.sqrt(hd)).astype(np.float32)
    dy = r.standard_normal((bs, s, d)).astype(np.float32)
    y_o, c_o, carried_o = ML.level_forward(p, cfg, x, m0)
    g_o, dx_o = ML.level_backward(p, cfg, c_o, dy, x)
    lp = MemoryLevelParams(*[dev(p[n]) for n in NAMES])
    ctx, emb = dev(m0), dev(x.reshape(bs * s, d))
    y, cache = GL.gpu_memory_forward(lp, cfg, emb, ctx, s, d, bs)
    grads = GL.LevelGrads.zeros(d)
    d_emb = GL.gpu_memory_backward(lp, cfg, cache, dev(dy.reshape(bs * s, d)), emb, grads, s, d, bs)
    torch.cuda.synchronize()
    assert cache.kind == "TitansMlp" and cache.d_hidden == dh
    out = dict(y=(host(y).reshape(bs, s, d), y_o), cache=(cache, c_o), carried=(host(ctx), carried_o),
               grads=(grads, g_o), d_x=(host(d_emb).reshape(bs, s, d), dx_o))
    check(out, "TitansMlp", tol=2e-4, has_eta=True)
    assert cache.dgd_delta_norm(s, d, 1, 1) == 0.0
    with pytest.raises(ValueError):
        GL.gpu_memory_forward(lp, GL.LevelConfig("titans", nh, hd, memory_layers=2, checkpoint_interval=4), emb, ctx, s,
                              d, bs)


@pytest.mark.parametrize("rule", ["moneta", "yaad"])
@pytest.mark.parametrize("s,d,dh", [(7, 16, 24), (12, 8, 32)])
def test_mlp_memories_at_model_width(rule, s, d, dh):
    """MONETA / YAAD levels (gpu_forward.rs:1729-1852, gpu_backward.rs:1635-1733): one sequence, context_m = [W1|W2]."""
    cfg = GL.LevelConfig(rule, 1, d, d_hidden=dh, lp_p=3.0, sign_sharpness=8.0, lambda_2=0.02, delta=0.5,
                         lambda_local=0.05, theta_ceil=0.4)
    r = np.random.default_rng(50 + s)
    p = params(d, 51)
    x = (r.standard_normal((1, s, d)) / np.sqrt(d)).astype(np.float32)
    w1 = (r.standard_normal((dh, d)) / np.sqrt(d)).astype(np.float32)
    w2 = (r.standard_normal((d, dh)) / np.sqrt(dh)).astype(np.float32)
    dy = r.standard_normal((1, s, d)).astype(np.float32)
    y_o, c_o, (w1_f, w2_f) = ML.level_forward(p, cfg, x, (w1, w2))
    g_o, dx_o = ML.level_backward(p, cfg, c_o, dy, x)
    lp = MemoryLevelParams(*[dev(p[n]) for n in NAMES])
    ctx = dev(np.concatenate([w1.ravel(), w2.ravel()]))
    emb = dev(x.reshape(s, d))
    y, cache = GL.gpu_memory_forward(lp, cfg, emb, ctx, s, d, 1)
    grads = GL.LevelGrads.zeros(d)
    d_emb = GL.gpu_memory_backward(lp, cfg, cache, dev(dy.reshape(s, d)), emb, grads, s, d, 1)
    torch.cuda.synchronize()
    assert cache.kind == "Mlp" and (cache.w1_boundary is not None) == (rule == "yaad")
    assert_close("y", host(y), y_o[0], 2e-4)
    assert_close("w1_states", host(cache.w1_states).reshape(c_o["w1_states"].shape), c_o["w1_states"], 2e-4)
    assert_close("w2_states", host(cache.w2_states).reshape(c_o["w2_states"].shape), c_o["w2_states"], 2e-4)
    got = host(ctx)
    assert_close("carried W1", got[:dh * d].reshape(dh, d), w1_f, 2e-4)
    assert_close("carried W2", got[dh * d:].reshape(d, dh), w2_f, 2e-4)
    for n in ("w_k", "w_v", "w_q"):
        assert_close("d_" + n, host(getattr(grads, f"d_{n}_mem")), g_o[n], 5e-4)
    for n in ("alpha", "theta"):
        assert_close("d_w_" + n, host(getattr(grads, "d_w_" + n)), g_o["w_" + n], 5e-4)
        assert_close("d_b_" + n, host(getattr(grads, "d_b_" + n)), g_o["b_" + n], 5e-4)
    assert_close("d_embedded", host(d_emb), dx_o[0], 5e-4)
    with pytest.raises(ValueError):
        GL.gpu_memory_forward(lp, cfg, dev(np.zeros((2 * s, d), np.float32)), ctx, s, d, 2)
    with pytest.raises(ValueError):
        GL.gpu_memory_forward(lp, cfg, emb, dev(np.zeros(10, np.float32)), s, d, 1)


def test_swiglu_level():
    """The stateless MLP level (gpu_forward.rs:1705-1727, gpu_backward.rs:1736-1760): no memory, direct gradients."""
    bs, s, d, inter = 2, 9, 16, 40
    r = np.random.default_rng(70)
    f = np.float32
    p = dict(gate_proj=(r.standard_normal((inter, d)) / np.sqrt(d)).astype(f),
             up_proj=(r.standard_normal((inter, d)) / np.sqrt(d)).astype(f),
             down_proj=(r.standard_normal((d, inter)) / np.sqrt(inter)).astype(f))
    x, dy = r.standard_normal((bs, s, d)).astype(f), r.standard_normal((bs, s, d)).astype(f)
    cfg = GL.LevelConfig("swiglu", 2, 8, intermediate_size=inter)
    y_o, c_o, _ = ML.level_forward(p, cfg, x, None)
    g_o, dx_o = ML.level_backward(p, cfg, c_o, dy, x)
    lp = GL.SwiGluLevelParams(dev(p["gate_proj"]), dev(p["up_proj"]), dev(p["down_proj"]))
    ctx = dev(np.full((4, 64), 7.0, f))
    emb = dev(x.reshape(bs * s, d))
    y, cache = GL.gpu_memory_forward(lp, cfg, emb, ctx, s, d, bs)
    grads = GL.LevelGrads.zeros(d, intermediate=inter)
    d_emb = GL.gpu_memory_backward(lp, cfg, cache, dev(dy.reshape(bs * s, d)), emb, grads, s, d, bs)
    torch.cuda.synchronize()
    assert cache.kind == "SwiGlu" and cache.alpha_stats(0.0) is None
    assert np.all(host(ctx) == 7.0), "a SwiGLU level leaves context_m alone"
    assert_close("y", host(y).reshape(bs, s, d), y_o, 1e-4)
    assert_close("d_x", host(d_emb).reshape(bs, s, d), dx_o, 1e-4)
    for n in ("gate_proj", "up_proj", "down_proj"):
        assert_close("d_" + n, host(getattr(grads, "d_" + n)), g_o[n], 1e-4)
