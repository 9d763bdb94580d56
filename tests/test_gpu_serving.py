"""GPU parity of the cached generation path (nl_hecate_amd.serving: GpuKVCache, gpu_prefill_forward,
gpu_single_token_forward as in core/src/gpu_forward.rs:2979-3492) against its CPU composition
(oracle/serving.py).  The attention branch stores bf16: logits at the bf16 bar (2e-2 relative); cache contents
bit for bit; memories 1e-4."""
import types

import numpy as np
import pytest
import torch

from nl_hecate_amd import serving as SG
from nl_hecate_amd.cms import ContextState, Pulse
from nl_hecate_amd.mag_layer import MemoryLevelParams
from nl_hecate_amd.memory_level import LevelConfig
from oracle import pyoracle as orc
from oracle import serving as SV
from tests.gpu_util import assert_close, dev, host
from tests.test_gpu_memory_level import NAMES
from tests.test_oracle_serving import model

pytestmark = pytest.mark.gpu
f32 = np.float32


def bits(t):
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def gpu_params(p):
    lv = [MemoryLevelParams(*[dev(l[n]) for n in NAMES]) for l in p["levels"]]
    return SG.GpuMAGParams(dev(p["w_embed"]), dev(p["w_q"]), dev(p["w_k"]), dev(p["w_v"]), dev(p["w_o"]),
                           dev(p["w_unembed"]), lv)


def test_kv_cache_append_persistent_refresh_reset():
    d, r = 16, np.random.default_rng(0)
    c = SG.GpuKVCache(10, d, 4)
    k, v = r.standard_normal((3, d)).astype(f32), r.standard_normal((3, d)).astype(f32)
    c.append_f32(dev(k), dev(v), 3)
    k2, v2 = r.standard_normal((4, d)).astype(f32), r.standard_normal((4, d)).astype(f32)
    c.append_f32(dev(k2), dev(v2), 4)
    assert c.len == 7
    assert np.array_equal(bits(c.k_cache_bf16)[:7], orc.f32_to_bf16(np.concatenate([k, k2])))
    assert np.array_equal(bits(c.v_cache_bf16)[:7], orc.f32_to_bf16(np.concatenate([v, v2])))
    assert not bits(c.k_cache_bf16)[7:].any()
    with pytest.raises(OverflowError):
        c.append_f32(dev(k2), dev(v2), 4)
    with pytest.raises(ValueError):
        SG.GpuKVCache(100, d, 2).append_f32(dev(k), dev(v), 3)
    # persistent prefix: projections of the persistent tokens at positions [0, n_p)
    pt = r.standard_normal((2, d)).astype(f32)
    wk, wv = r.standard_normal((d, d)).astype(f32) * 0.3, r.standard_normal((d, d)).astype(f32) * 0.3
    with pytest.raises(RuntimeError):
        c.prepopulate_persistent(dev(pt), dev(wk), dev(wv), 2, d)
    c.reset()
    assert c.len == 0
    c.prepopulate_persistent(dev(pt), dev(wk), dev(wv), 2, d)
    assert c.len == 2
    want_k = orc.bf16_to_f32(orc.f32_to_bf16((pt @ wk.T).astype(f32)))
    assert np.abs(orc.bf16_to_f32(bits(c.k_cache_bf16)[:2]) - want_k).max() <= 2 ** -7 * np.abs(want_k).max()
    c.append_f32(dev(k), dev(v), 3)
    c.refresh_persistent(dev(2 * pt), dev(wk), dev(wv), 2, d)
    assert c.len == 5
    got = orc.bf16_to_f32(bits(c.v_cache_bf16)[:2])
    want_v = 2 * (pt @ wv.T)
    assert np.abs(got - want_v).max() <= 2 ** -7 * np.abs(want_v).max()
    assert np.array_equal(bits(c.k_cache_bf16)[2:5], orc.f32_to_bf16(k))
    with pytest.raises(RuntimeError):
        SG.GpuKVCache(10, d, 4).refresh_persistent(dev(pt), dev(wk), dev(wv), 2, d)


CASES = [  # rule, k, active, n_persistent, nh, hd, window, s, extra
    ("delta", 1, [True], 0, 2, 8, 6, 12, 6),
    ("delta", 2, [True, False], 0, 2, 16, 5, 9, 5),
    ("titans", 3, [True, True, False], 2, 2, 8, 4, 10, 6),
    ("hebbian", 2, [False, True], 0, 1, 16, 8, 7, 4),
    ("dgd", 4, [True, False, True, False], 1, 2, 8, 16, 8, 3),
]


@pytest.mark.parametrize("rule,k,active,n_persistent,nh,hd,window,s,extra", CASES)
def test_prefill_then_decode(rule, k, active, n_persistent, nh, hd, window, s, extra):
    d, v = nh * hd, 23
    p = model(d, v, k, 60 + k + hd)
    lcfgs = [LevelConfig(rule, nh, hd) for _ in range(k)]
    ocfg = types.SimpleNamespace(d_model=d, num_heads=nh, head_dim=hd, window_size=window, n_persistent=n_persistent,
                                 levels=lcfgs)
    cfg = SG.ServeConfig(d, v, nh, hd, window, s, lcfgs, n_persistent=n_persistent, decode_tokens=extra)
    r = np.random.default_rng(5)
    ids = r.integers(0, v, s + extra)
    mem0 = [(0.2 * r.standard_normal((nh, hd, hd))).astype(f32) for _ in range(k)]
    pulse = Pulse(0, list(active))
    gp = gpu_params(p)
    ctx = ContextState([dev(m.reshape(nh, hd * hd)) for m in mem0])
    logits, kv = SG.gpu_prefill_forward(gp, cfg, ids, pulse, ctx)
    want, mem, kc, vc = SV.forward_all(p, ocfg, ids[:s], active, mem0)
    scale = np.abs(want).max()
    assert np.abs(logits - want[s - 1]).max() <= 2e-2 * scale
    assert kv.len == s and kv.max_len == s + extra
    # the cache holds bf16(k), bf16(v) of fp32 projections: equal up to one bf16 step where the GEMMs round apart
    for got, ref in ((kv.k_cache_bf16, kc), (kv.v_cache_bf16, vc)):
        a, b = orc.bf16_to_f32(bits(got)[:s]), orc.bf16_to_f32(ref)
        assert np.abs(a - b).max() <= 2 ** -7 * np.abs(b).max()
    ws = SG.DecodeWorkspace(d, v)
    for i in range(extra):
        step = SG.gpu_single_token_forward(gp, cfg, int(ids[s + i]), pulse, ctx, kv, ws)
        ref, mem, kc, vc = SV.single_token(p, ocfg, int(ids[s + i]), active, mem, kc, vc)
        assert np.abs(step - ref).max() <= 2e-2 * scale, i
        assert kv.len == s + i + 1
    for lv in range(k):
        assert_close(f"memory[{lv}]", host(ctx.memory[lv]).reshape(mem[lv].shape), mem[lv], 1e-4)
    with pytest.raises(OverflowError):
        SG.gpu_single_token_forward(gp, cfg, 0, pulse, ctx, kv, ws)
    with pytest.raises(ValueError):
        SG.gpu_single_token_forward(gp, cfg, v, pulse, ctx, kv, ws)


def test_decode_needs_a_prefilled_cache():
    d, v = 16, 7
    p = model(d, v, 1, 3)
    cfg = SG.ServeConfig(d, v, 2, 8, 4, 4, [LevelConfig("delta", 2, 8)])
    with pytest.raises(RuntimeError):
        SG.gpu_single_token_forward(gpu_params(p), cfg, 1, Pulse(0, [True]), ContextState([dev(np.zeros((2, 64), f32))]),
                                    SG.GpuKVCache(8, d, 1), SG.DecodeWorkspace(d, v))


def test_frozen_mlp_memory_levels_follow_the_reference():
    """gpu_forward.rs:32-57, 3255-3265: a frozen MONETA / YAAD level contributes zeros (its context memory is the flat
    [W1 | W2] block, which the matrix read must not interpret); a frozen two-layer Titans memory is refused."""
    nh, hd, window, s, extra, v, k = 2, 8, 6, 9, 3, 19, 2
    d = nh * hd
    p = model(d, v, k, 77)
    r = np.random.default_rng(9)
    ids = r.integers(0, v, s + extra)
    active = [True, False]
    for frozen_rule in ("moneta", "yaad"):
        lcfgs = [LevelConfig("delta", nh, hd), LevelConfig(frozen_rule, nh, hd, d_hidden=12)]
        ocfg = types.SimpleNamespace(d_model=d, num_heads=nh, head_dim=hd, window_size=window, n_persistent=0, levels=lcfgs)
        cfg = SG.ServeConfig(d, v, nh, hd, window, s, lcfgs, decode_tokens=extra)
        mem0 = [(0.2 * r.standard_normal((nh, hd, hd))).astype(f32), r.standard_normal(2 * 12 * d).astype(f32)]
        ctx = ContextState([dev(mem0[0].reshape(nh, hd * hd)), dev(mem0[1])])
        gp = gpu_params(p)
        logits, kv = SG.gpu_prefill_forward(gp, cfg, ids, Pulse(0, active), ctx)
        want, mem, kc, vc = SV.forward_all(p, ocfg, ids[:s], active, mem0)
        scale = np.abs(want).max()
        assert np.abs(logits - want[s - 1]).max() <= 2e-2 * scale
        ws = SG.DecodeWorkspace(d, v)
        for i in range(extra):
            step = SG.gpu_single_token_forward(gp, cfg, int(ids[s + i]), Pulse(0, active), ctx, kv, ws)
            ref, mem, kc, vc = SV.single_token(p, ocfg, int(ids[s + i]), active, mem, kc, vc)
            assert np.abs(step - ref).max() <= 2e-2 * scale, i
        assert np.array_equal(host(ctx.memory[1]), mem0[1]), "a frozen level's memory is not touched"
    lcfgs = [LevelConfig("delta", nh, hd), LevelConfig("titans", nh, hd, memory_layers=2)]
    cfg = SG.ServeConfig(d, v, nh, hd, window, s, lcfgs, decode_tokens=extra)
    ctx = ContextState([dev(np.zeros((nh, hd * hd), f32)), dev(np.zeros(8, f32))])
    with pytest.raises(RuntimeError, match="Frozen TitansLMM MLP"):
        SG.gpu_prefill_forward(gpu_params(p), cfg, ids, Pulse(0, active), ctx)
    with pytest.raises(AssertionError, match="residual"):
        SG.gpu_prefill_forward(gpu_params(p), SG.ServeConfig(d, v, nh, hd, window, s, lcfgs[:1], residual=True), ids,
                               Pulse(0, [True]), ctx)
