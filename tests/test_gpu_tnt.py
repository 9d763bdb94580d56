"""GPU parity of the TNT level on device buffers (nl_hecate_amd.tnt: gpu_tnt_forward and the TNT backward of the
reference, core/src/gpu_forward.rs:1878-2293, gpu_backward.rs:1201-1632) against its CPU composition
(oracle/memory_level.py tnt_forward / tnt_backward), float32, relative 1e-4."""
import numpy as np
import pytest
import torch

from nl_hecate_amd import memory_level as GL
from nl_hecate_amd import tnt as TN
from nl_hecate_amd.mag_layer import MemoryLevelParams
from oracle import memory_level as ML
from tests.gpu_util import assert_close, dev, host
from tests.test_gpu_memory_level import NAMES, params

pytestmark = pytest.mark.gpu
f32 = np.float32


def run(cfg, s, cg, cl, seed, max_retained=None, per_head=False):
    nh, hd = cfg.num_heads, cfg.head_dim
    d = nh * hd
    r = np.random.default_rng(seed)
    p = params(d, seed + 1)
    x = (r.standard_normal((s, d)) / np.sqrt(d)).astype(f32)
    m0 = (0.3 * r.standard_normal((nh, hd, hd))).astype(f32)
    dy = r.standard_normal((s, d)).astype(f32)
    y_o, shards, m_fin = ML.tnt_forward(p, cfg, x, m0, cg, cl)
    n_shards = len(shards)
    first = 0 if max_retained is None else max(0, n_shards - max(1, max_retained))
    g_o, dx_o = ML.tnt_backward(p, cfg, shards, dy, x, cl, first_retained=first, per_head_memory_gradient=per_head)
    lp = MemoryLevelParams(*[dev(p[n]) for n in NAMES])
    ctx, emb = dev(m0.reshape(nh, hd * hd)), dev(x)
    y, cache = TN.gpu_tnt_forward(lp, cfg, emb, ctx, s, d, 1, TN.ParallelConfig(cg, cl), max_retained)
    grads = GL.LevelGrads.zeros(d)
    d_emb = TN.gpu_tnt_backward(lp, cfg, cache, dev(dy), emb, grads, s, d, 1, per_head_memory_gradient=per_head)
    torch.cuda.synchronize()
    assert cache.total_shards == n_shards and cache.first_retained_shard == first
    assert len(cache.shard_inner_caches) == n_shards - first and len(cache.k_summaries) == n_shards
    assert_close("y", host(y), y_o)
    assert_close("global memory", host(ctx).reshape(m_fin.shape), m_fin)
    for i, c in enumerate(shards):
        assert_close(f"k summary {i}", host(cache.k_summaries[i]), c["summary"].reshape(-1))
        assert_close(f"v summary {i}", host(cache.v_summaries[i]), c["summary"].reshape(-1))
    titans = cfg.memory_rule == "titans"
    for n in ("w_k", "w_v", "w_q"):
        assert_close("d_" + n, host(getattr(grads, f"d_{n}_mem")), g_o[n])
    for n in ["alpha", "theta"] + (["eta"] if titans else []):
        assert_close("d_w_" + n, host(getattr(grads, "d_w_" + n)), g_o["w_" + n])
        assert_close("d_b_" + n, host(getattr(grads, "d_b_" + n)), g_o["b_" + n])
    assert_close("d_embedded", host(d_emb), dx_o)
    return cache


@pytest.mark.parametrize("rule", ["delta", "titans"])
@pytest.mark.parametrize("nh,hd,s,cg,cl", [(1, 8, 24, 8, 4), (2, 8, 22, 8, 3), (1, 16, 9, 16, 4), (3, 8, 20, 5, 5),
                                           (2, 16, 16, 8, 8)])
def test_forward_and_backward_match_the_composition(rule, nh, hd, s, cg, cl):
    """Ragged last shards, padded last local chunks, several heads (where the reference's backward adds every
    head's initial-memory gradient to head 0: the composition does the same)."""
    cache = run(GL.LevelConfig(rule, nh, hd), s, cg, cl, 400 + s + hd)
    inner = cache.shard_inner_caches[0]
    assert inner.kind == ("Titans" if rule == "titans" else "Delta") and not inner.proxy
    assert inner.m_states.shape == (nh * -(-min(cg, s) // cl), cl + 1, hd * hd)


@pytest.mark.parametrize("rule", ["delta", "titans"])
@pytest.mark.parametrize("nh,hd,s,cg,cl", [(2, 8, 22, 8, 3), (3, 8, 20, 5, 5)])
def test_per_head_attribution_of_the_initial_memory_gradients(rule, nh, hd, s, cg, cl):
    """The option that sends every local chain's initial-memory gradient to its own head (the gradient of the forward
    for several heads: central differences of the float64 composition confirm it, tests/test_oracle_memory_level.py);
    the default above is the reference's attribution to head 0."""
    run(GL.LevelConfig(rule, nh, hd), s, cg, cl, 500 + s + hd, per_head=True)


@pytest.mark.parametrize("rule", ["delta", "titans"])
def test_proxy_levels_keep_final_states_only(rule):
    cache = run(GL.LevelConfig(rule, 2, 8, proxy=True), 18, 6, 3, 431)
    inner = cache.shard_inner_caches[0]
    assert inner.proxy and inner.m_states.shape == (2 * 2, 64)
    assert inner.dgd_delta_norm(3, 8, 1, 1) == 0.0


def test_clamps_clip_and_norm_bound():
    run(GL.LevelConfig("titans", 2, 8, alpha_floor=0.22, alpha_ceil=0.3, theta_ceil=0.2, error_clip=0.7,
                       m_norm_max=1.2), 20, 8, 4, 440)


@pytest.mark.parametrize("max_retained", [1, 2])
def test_rolling_window_of_inner_caches(max_retained):
    """Shards whose inner caches were dropped only pass the global memory's gradient on (spec 25 of the reference)."""
    run(GL.LevelConfig("delta", 1, 8), 30, 6, 3, 450, max_retained=max_retained)


def test_delta_norm_and_argument_errors():
    cfg = GL.LevelConfig("delta", 1, 8)
    cache = run(cfg, 12, 4, 4, 460)
    worst = max(c.dgd_delta_norm(4, 8, 1, 1) for c in cache.shard_inner_caches)
    assert cache.dgd_delta_norm(12, 8, 1, 1) == worst and worst > 0.0
    lp = MemoryLevelParams(*[dev(params(8, 1)[n]) for n in NAMES])
    z, ctx = dev(np.zeros((4, 8), f32)), dev(np.zeros((1, 64), f32))
    with pytest.raises(ValueError):
        TN.gpu_tnt_forward(lp, cfg, z, ctx, 2, 8, 2, TN.ParallelConfig(2, 2))
    with pytest.raises(ValueError):
        TN.gpu_tnt_forward(lp, GL.LevelConfig("hebbian", 1, 8), z, ctx, 4, 8, 1, TN.ParallelConfig(2, 2))
    with pytest.raises(ValueError):
        TN.gpu_tnt_forward(lp, cfg, z, dev(np.zeros(10, f32)), 4, 8, 1, TN.ParallelConfig(2, 2))
